"""Branches of the kernels and of the wrapper that the broader GPU tests do not reach: the decision
kernel over more chunks than it stages, a refresh workgroup that takes several pieces, and a wrapper
step with more hyper records than the update launch's arguments or the control block can carry."""
import math

import numpy as np
import pytest
import torch

import elixir_amd as ea
from elixir_amd import _abi
from elixir_amd.chunk import DeviceTable
from elixir_amd.hybrid_adam import make_hyper_record
from oracle import oracle as O

from helpers import CODE, build_workload, compare_state, refresh_oracle_grads, to_np

pytestmark = pytest.mark.gpu
DEV = 'cuda'
REC = _abi.STATS_DTYPE.itemsize
HSZ = _abi.HYPER_DTYPE.itemsize


@pytest.mark.parametrize('overflow', [False, True])
@pytest.mark.parametrize('n', [1500, 4000])
def test_finish_decide_over_more_chunks_than_it_stages(n, overflow):
    """The decision workgroup stages 1024 per-chunk records in LDS and reads the rest from memory, both
    in its decision loop and when it copies the records into the report: 1,500 and 4,000 tiny chunks
    (two partials each; with ``overflow`` an inf in chunk 1,400; clipping on) against elx_grad_stats_mt
    followed by elx_decide on the same gradients -- identical records, decision, gate words and report."""
    rng = np.random.default_rng(n)
    sizes = rng.integers(1, 400, n)
    starts = np.concatenate(([0], np.cumsum((sizes + 7) // 8 * 8)))    # every chunk starts on a 16-byte boundary
    gen = torch.Generator(device=DEV).manual_seed(n)
    g = (torch.randn(int(starts[-1]), generator=gen, device=DEV) * 2.0).half()
    if overflow:
        g[int(starts[1400]) + int(sizes[1400]) - 1] = float('inf')
    rows = np.zeros(n, dtype=_abi.CHUNK_DTYPE)
    rows['grad'] = g.data_ptr() + 2 * starts[:-1].astype(np.uint64)
    rows['n_alloc'] = rows['n_valid'] = sizes
    table = DeviceTable(rows, torch.device(DEV, 0))
    stream = torch.cuda.current_stream().cuda_stream
    bpc, n_hyp, loss_scale, max_norm = 2, 3, 64.0, 0.75
    hyp_host = np.concatenate([make_hyper_record(1e-3 * (k + 1), 0.9, 0.999, 1e-8, 0.01 * k, 1 + k, True, True)
                               for k in range(n_hyp)])
    H = _abi.max_ctl_hypers()

    ws = torch.empty((n * bpc + n) * REC, dtype=torch.uint8, device=DEV)
    _abi.grad_stats_mt(table.ptr, n, _abi.ELX_F16, bpc, ws.data_ptr(), ws.data_ptr() + n * bpc * REC, False, stream)
    hyp_a = torch.from_numpy(hyp_host.view(np.uint8).copy()).to(DEV)
    dec_a = torch.zeros(32, dtype=torch.uint8, device=DEV)
    _abi.decide(ws.data_ptr() + n * bpc * REC, n, loss_scale, max_norm, True, hyp_a.data_ptr(), n_hyp, dec_a.data_ptr(),
                stream)

    ctl_head, rep_head = _abi.STEP_CTL_DTYPE.itemsize, _abi.STEP_REPORT_DTYPE.itemsize
    ctl = torch.zeros(ctl_head + H * HSZ, dtype=torch.uint8, pin_memory=True)
    cb = ctl.numpy()
    cb[:ctl_head].view(_abi.STEP_CTL_DTYPE)[0] = (loss_scale, max_norm, 1, n_hyp, 4242)
    cb[ctl_head:ctl_head + hyp_host.nbytes] = hyp_host.view(np.uint8).reshape(-1)
    report = torch.zeros(rep_head + n * REC, dtype=torch.uint8, pin_memory=True)
    partials = torch.empty(n * bpc * REC, dtype=torch.uint8, device=DEV)
    stats_b = torch.zeros(n * REC, dtype=torch.uint8, device=DEV)
    hyp_b = torch.full((H * HSZ, ), 0xEE, dtype=torch.uint8, device=DEV)
    dec_b = torch.zeros(32, dtype=torch.uint8, device=DEV)
    counter = torch.zeros(4, dtype=torch.int32, device=DEV)
    _abi.grad_partials_mt(table.ptr, n, _abi.ELX_F16, bpc, partials.data_ptr(), False, stream)
    _abi.finish_decide(partials.data_ptr(), n, bpc, stats_b.data_ptr(), ctl.data_ptr(), hyp_b.data_ptr(), H,
                       dec_b.data_ptr(), report.data_ptr(), counter.data_ptr(), stream)
    torch.cuda.synchronize()

    want_stats = ws[n * bpc * REC:].cpu().numpy()
    assert want_stats.tobytes() == stats_b.cpu().numpy().tobytes()
    assert dec_a.cpu().numpy().tobytes() == dec_b.cpu().numpy().tobytes()
    assert hyp_a.cpu().numpy().tobytes() == hyp_b[:n_hyp * HSZ].cpu().numpy().tobytes()
    assert bool((hyp_b[n_hyp * HSZ:] == 0xEE).all())
    rb = report.numpy()
    rh = rb[:rep_head].view(_abi.STEP_REPORT_DTYPE)[0]
    assert rh['seq'] == 4242 and rh['n_chunks'] == n and rh['status'] == 0 and bool(rh['skip']) == overflow
    assert rb[:32].tobytes() == dec_b.cpu().numpy().tobytes()
    assert rb[rep_head:].tobytes() == want_stats.tobytes()          # every record, staged or not, reached the host
    assert int(counter[0]) == 0
    recs = want_stats.view(_abi.STATS_DTYPE)
    assert int(recs['overflow'].sum()) == (1 if overflow else 0) and (not overflow or recs['overflow'][1400] == 1)
    # the decision itself, from the records, in the reference's float64 arithmetic
    if not overflow:
        l2 = [float(np.float32(np.sqrt(x)))**2 for x in recs['sumsq']]
        norm = O.global_norm(l2)
        assert float(rh['total_norm']) == norm
        assert float(rh['combined_scale']) == float(ea.calc_combined_scale(loss_scale, norm, max_norm, True))


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_refresh_workgroups_take_several_pieces(oracle, dtype):
    """elx_writeback_mt with fewer workgroups per record than the record has pieces: three workgroups
    walk the 100 pieces of the first record (the last piece partial) with the stride of the grid, and the
    5 pieces of the second.  Every element equals the oracle's round-to-nearest-even cast."""
    piece = _abi.refresh_piece_elems()
    sizes = [100 * piece - 77, 5 * piece]
    gen = torch.Generator(device=DEV).manual_seed(9)
    masters = [torch.randn(k, generator=gen, device=DEV) * 3.0 for k in sizes]
    masters[0][:4] = torch.tensor([65504.0, 65520.0, -0.0, 1e-8], device=DEV)
    outs = [torch.full((k, ), 7.0, dtype=dtype, device=DEV) for k in sizes]
    rows = np.zeros(2, dtype=_abi.CHUNK_DTYPE)
    for i in range(2):
        rows[i]['lowp_out'], rows[i]['master'], rows[i]['n_alloc'] = outs[i].data_ptr(), masters[i].data_ptr(), sizes[i]
    table = DeviceTable(rows, torch.device(DEV, 0))
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check('elx_writeback_mt', _abi.load().elx_writeback_mt(table.ptr, 2, CODE[dtype], 3, 0, stream))
    torch.cuda.synchronize()
    for out, master in zip(outs, masters):
        want = oracle.writeback(to_np(master), CODE[dtype])
        got = to_np(out)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def _groups_one_per_tensor(entries):
    """Every tensor a parameter group of its own, each with its own learning rate (layer-wise decay) and
    one of three weight decays."""
    return [dict(params=[p], lr=1e-3 * (0.97**i), weight_decay=(0.0, 0.01, 0.1)[i % 3]) for i, (_, _, p) in enumerate(entries)]


@pytest.mark.parametrize('cap', [None, 64], ids=['control_block', 'host_fallback'])
@pytest.mark.parametrize('gated', [True, False])
def test_seventy_param_groups(oracle, monkeypatch, gated, cap):
    """optimizer.py:246-265: the group hyper-parameters survive untouched, however many groups there
    are.  70 tensors in 70 groups (distinct learning rates, three weight decays) over two fp16 chunks,
    clipping on, three steps of which the second overflows.  Decided on the device through the control
    block; with the device's capacity forced down to 64 records, decided on the host from the partials
    the early stats launch left (the gradients are read once all the same); and with ``gated_step`` off.
    Every step issues exactly one stats launch; the results follow the oracle."""
    dtype = torch.float16
    named = [(f't{i}', (257 + 61 * i, )) for i in range(70)]
    total = sum(s[0] for _, s in named)
    module, opt, ochunks = build_workload(named, 1 << int(math.ceil(math.log2(total / 2 + 20000))), dtype, seed=41,
                                          grad_std=2e-2, loss_scale=128.0, groups_of=_groups_one_per_tensor,
                                          max_norm=1.0, initial_scale=128.0, hysteresis=1)
    assert len(module.param_chunks) == 2 and len(opt.param_groups) == 70
    assert len({g['lr'] for g in opt.param_groups}) == 70
    opt.gated_step = gated
    if cap is not None:
        opt.max_device_hypers = cap
    scaler = O.DynamicGradScalerOracle(initial_scale=128.0, min_scale=1, max_scale=2**24, hysteresis=1)
    launches = []
    for name in ('grad_partials_mt', 'grad_stats_mt', 'grad_stats'):
        real = getattr(_abi, name)
        monkeypatch.setattr(_abi, name, lambda *a, _real=real, _name=name, **k: (launches.append(_name), _real(*a, **k))[1])
    updates = []
    for name in ('adam_step_gated_mt', 'adam_step_mt', 'adam_step_put_mt'):
        real = getattr(_abi, name)
        monkeypatch.setattr(_abi, name, lambda *a, _real=real, _name=name, **k: (updates.append(_name), _real(*a, **k))[1])
    gen = torch.Generator(device=DEV).manual_seed(42)
    for step in range(3):
        if step:
            for pc in module.param_chunks:
                g = torch.randn(pc.shard_size, generator=gen, device=DEV) * (2e-2 * opt.loss_scale)
                g[pc.utilized_size:] = 0
                pc.shard.copy_(g.to(dtype))
                pc.invalidate_stats()
            if step == 1:
                module.param_chunks[1].shard[17] = float('-inf')
            refresh_oracle_grads(module, ochunks)
        launches.clear()
        updates.clear()
        opt.mark_gradients_scaled()
        assert len(opt.optim._prepared.hyper_host) == 70
        opt.step()
        assert len(launches) == 1, launches                       # one pass over the gradients per step
        info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=1.0)
        assert opt.last_step_info['found_inf'] == info['found_inf'] == (step == 1)
        assert opt.loss_scale == info['loss_scale']
        if step == 1:
            assert updates in ([], ['adam_step_gated_mt'])        # skipped: the host-decided step launches no update
        else:
            assert updates == (['adam_step_gated_mt'] if gated and cap is None else ['adam_step_mt'])
            assert math.isclose(opt.last_step_info['combined_scale'], info['combined_scale'], rel_tol=1e-6)
        compare_state(module, opt, ochunks, dtype, rtol=1e-6, atol_p=1e-9, atol_m=1e-8, atol_v=1e-10, tag=f'step {step}')
    assert [g['lr'] for g in opt.param_groups] == [1e-3 * (0.97**i) for i in range(70)]
    assert opt.loss_scale == 64.0


def test_more_groups_than_the_control_block_holds(oracle):
    """300 groups: beyond the 256 records of the control block, the step is decided on the host from
    the one pass over the gradients that went out early; identical bits to the same step with
    ``gated_step`` off."""
    dtype = torch.bfloat16
    named = [(f't{i}', (64 + 8 * (i % 17), )) for i in range(300)]
    states = []
    for gated in (True, False):
        module, opt, ochunks = build_workload(named, 1 << 14, dtype, seed=43, grad_std=1e-2, loss_scale=1.0,
                                              groups_of=_groups_one_per_tensor, max_norm=0.5)
        assert len(opt.param_groups) == 300 > _abi.max_ctl_hypers()
        opt.gated_step = gated
        opt.mark_gradients_scaled()
        opt.step()
        info = O.reference_step(ochunks, CODE[dtype], O.ConstantGradScalerOracle(1.0), max_norm=0.5)
        assert opt.last_step_info['found_inf'] is False
        assert math.isclose(opt.last_step_info['combined_scale'], info['combined_scale'], rel_tol=1e-6)
        compare_state(module, opt, ochunks, dtype, rtol=1e-6, atol_p=1e-9, atol_m=1e-8, atol_v=1e-10)
        states.append([(pc.shard.clone(), pc.paired_chunk.shard.clone(), *[t.clone() for t in
                                                                            opt._binding.moments(pc.paired_chunk)])
                       for pc in module.param_chunks])
    for a, b in zip(*states):
        for x, y in zip(a, b):
            assert torch.equal(x.view(torch.int16) if x.dtype == dtype else x, y.view(torch.int16) if y.dtype == dtype else y)


@pytest.mark.parametrize('n_groups', [1, 2])
def test_standalone_steps_over_unchanged_buffers_take_the_steady_path(oracle, monkeypatch, n_groups):
    """A standalone HybridAdam whose parameters and gradient buffers stay where they are (the gradients
    are rewritten in place) repeats the launch of the step before with new hyper records only.  Twelve
    steps with a learning rate that changes every step and a divisor that changes too: every step after
    the first goes that way, and master / exp_avg / exp_avg_sq have the oracle's bits after each.  A step
    count edited behind the optimizer's back, a gradient that moves, a loaded state, a moment that moves and a
    replaced state entry each send one step through the full preparation again -- with the right result."""
    import elixir_amd.hybrid_adam as H
    sizes = [50_001, 4_097][:n_groups]
    torch.manual_seed(3)
    params = [torch.nn.Parameter((torch.randn(n) * 0.02).to(DEV)) for n in sizes]
    host = [(to_np(p.data).copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)) for p, n in zip(params, sizes)]
    steps = [0] * n_groups
    wds = [0.1, 0.0][:n_groups]
    opt = ea.HybridAdam([dict(params=[p], lr=1e-3 * (k + 1), weight_decay=wd) for k, (p, wd) in enumerate(zip(params, wds))])
    for p in params:
        p.grad = torch.zeros_like(p)
    taken = []
    real = H.HybridAdam._launch_steady
    monkeypatch.setattr(H.HybridAdam, '_launch_steady', lambda self, *a, **k: (taken.append(1), real(self, *a, **k))[1])
    gen = torch.Generator().manual_seed(4)

    def one_step(expect_steady):
        for k, group in enumerate(opt.param_groups):
            group['lr'] = 1e-3 * (k + 1) * (0.9**sum(steps))
        div = [-1.0, 4.0, 3.0][sum(steps) % 3]
        grads = [torch.randn(n, generator=gen) * 1e-2 * max(div, 1.0) for n in sizes]
        for p, g in zip(params, grads):
            p.grad.copy_(g.to(DEV))                      # the same buffer, new values
        before = len(taken)
        opt.step(div_scale=div)
        assert (len(taken) - before == 1) == expect_steady, (steps, expect_steady)
        for k, (p, g, (pn, mn, vn)) in enumerate(zip(params, grads, host)):
            steps[k] += 1
            oracle.adam(to_np(g), O.F32, pn, mn, vn, lr=opt.param_groups[k]['lr'], beta1=0.9, beta2=0.999, eps=1e-8,
                        weight_decay=wds[k], step=steps[k], adamw_mode=True, div_scale=div)
            st = opt.state[p]
            assert st['step'] == steps[k]
            for name, got, want in (('p', p.data, pn), ('m', st['exp_avg'], mn), ('v', st['exp_avg_sq'], vn)):
                assert np.array_equal(to_np(got).view(np.uint32), want.view(np.uint32)), (steps, name)

    one_step(False)
    for _ in range(11):
        one_step(True)
    # a step count changed behind the optimizer's back: the records must follow it
    opt.state[params[0]]['step'] = 40
    steps[0] = 40
    one_step(False)
    if n_groups == 1:
        one_step(True)
    else:
        one_step(False)    # two step counts now: every step is prepared in full (the records are matched to parameters)
    # a gradient that moved
    params[0].grad = torch.zeros_like(params[0])
    one_step(False)
    # a loaded state
    opt.load_state_dict(opt.state_dict())
    one_step(False)
    one_step(n_groups == 1)
    # a moment that moved (same values in a new tensor): the launch must follow it, as torch's optimizers would
    old_m = opt.state[params[0]]['exp_avg']
    opt.state[params[0]]['exp_avg'] = old_m.clone()
    frozen = old_m.clone()
    one_step(False)
    assert torch.equal(old_m, frozen)                  # the buffer left behind is no longer written
    one_step(n_groups == 1)
    # a state entry replaced as a whole
    st = opt.state[params[0]]
    opt.state[params[0]] = dict(step=st['step'], exp_avg=st['exp_avg'].clone(), exp_avg_sq=st['exp_avg_sq'].clone())
    one_step(False)
    one_step(n_groups == 1)


def test_decision_launch_arms_and_disarms_the_row_table_of_the_update():
    """elx_finish_decide_rows keeps the n_valid column of the gated update launch's row table: zeros when the
    step is skipped (an overflow, or an unusable control block), the counts of the untouched source table again
    at the first decision that lets a step happen -- so a table armed for a skip is disarmed by the next
    decision, whatever the host did in between -- and the word that says which of the two it holds.  Nothing else in the table changes, the source table never does, and the decision
    and report are those of elx_finish_decide.  Then the whole path: a skipped gated update over the armed
    table only refreshes, the step after it updates -- both equal to the same launches over an unarmed table."""
    stream = torch.cuda.current_stream().cuda_stream
    dev = torch.device(DEV, 0)
    tile = _abi.tile_elems()
    n_rows = 700                                       # more rows than the deciding workgroup has threads
    rng = np.random.default_rng(5)
    rows = np.zeros(n_rows, dtype=_abi.CHUNK_DTYPE)
    rows['n_alloc'] = rng.integers(1, 50_000, n_rows)
    rows['n_valid'] = (rows['n_alloc'] * rng.random(n_rows)).astype(np.uint64)
    for name in ('grad', 'lowp_out', 'master', 'm', 'v'):
        rows[name] = rng.integers(1, 1 << 40, n_rows) * 16
    rows['tile_begin'] = np.concatenate(([0], np.cumsum(-(-rows['n_alloc'] // tile))[:-1]))
    src, gated = DeviceTable(rows, dev), DeviceTable(rows, dev)
    H = _abi.max_ctl_hypers()
    ctl_head, rep_head = _abi.STEP_CTL_DTYPE.itemsize, _abi.STEP_REPORT_DTYPE.itemsize
    ctl = torch.zeros(ctl_head + H * HSZ, dtype=torch.uint8, pin_memory=True)
    head = ctl.numpy()[:ctl_head].view(_abi.STEP_CTL_DTYPE)
    report = torch.zeros(rep_head + 2 * REC, dtype=torch.uint8, pin_memory=True)
    stats = torch.zeros(2 * REC, dtype=torch.uint8, device=DEV)
    hyp = torch.zeros(H * HSZ, dtype=torch.uint8, device=DEV)
    dec = torch.zeros(32, dtype=torch.uint8, device=DEV)
    counter = torch.zeros(4, dtype=torch.int32, device=DEV)
    armed = torch.zeros(1, dtype=torch.int32, device=DEV)

    def decide(overflow, loss_scale=8.0):
        recs = np.zeros(2, dtype=_abi.STATS_DTYPE)
        recs['sumsq'] = [4.0, 9.0]
        recs['overflow'][1] = 1 if overflow else 0
        d_recs = torch.from_numpy(recs.view(np.uint8).copy()).to(DEV)
        head[0] = (loss_scale, 1.0, 0, 0, int(head['seq'][0]) + 1)
        _abi.finish_decide(d_recs.data_ptr(), 2, 1, stats.data_ptr(), ctl.data_ptr(), hyp.data_ptr(), H, dec.data_ptr(),
                           report.data_ptr(), counter.data_ptr(), stream, d_rows=src.ptr, d_gated_rows=gated.ptr,
                           n_rows=n_rows, d_armed=armed.data_ptr())
        torch.cuda.synchronize()
        assert int(armed[0]) == (1 if overflow or not loss_scale > 0 else 0)
        got = gated.dev.cpu().numpy().view(_abi.CHUNK_DTYPE)
        assert src.dev.cpu().numpy().tobytes() == rows.tobytes()           # the source table is never written
        for name in rows.dtype.names:
            if name != 'n_valid':
                assert np.array_equal(got[name], rows[name]), name
        rh = report.numpy()[:rep_head].view(_abi.STEP_REPORT_DTYPE)[0]
        assert rh['seq'] == head['seq'][0]
        return got['n_valid'].copy(), int(rh['skip']), int(rh['status'])

    valid, skip, status = decide(False)
    assert np.array_equal(valid, rows['n_valid']) and (skip, status) == (0, 0)
    valid, skip, status = decide(True)
    assert not valid.any() and (skip, status) == (1, 0)
    valid, skip, status = decide(True)                                     # armed twice in a row
    assert not valid.any() and skip == 1
    valid, skip, status = decide(False)                                    # disarmed by the next decision
    assert np.array_equal(valid, rows['n_valid']) and skip == 0
    valid, skip, status = decide(False, loss_scale=0.0)                    # an unusable control block: nothing may update
    assert not valid.any() and (skip, status) == (1, _abi.ELX_E_RANGE)
    valid, skip, status = decide(False)
    assert np.array_equal(valid, rows['n_valid']) and (skip, status) == (0, 0)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_skipped_step_over_the_armed_table_refreshes_everything_and_updates_nothing(oracle, dtype):
    """The wrapper's device-decided step with an overflow: master, exp_avg, exp_avg_sq and the step counts stay
    as they were, every element of every low-precision shard -- owned by a tensor or not, padding included,
    whatever sat there -- becomes the cast of its master value, and the clean step behind it updates as the
    oracle does."""
    module, opt, ochunks = build_workload([('a', (70_001, )), ('b', (33, 1000)), ('c', (5, )), ('d', (100_000, ))], 1 << 17,
                                          dtype, seed=51, grad_std=2e-2, loss_scale=256.0 if dtype == torch.float16 else 1.0,
                                          weight_decay=0.1, max_norm=1.0, initial_scale=256.0, hysteresis=1)
    if dtype == torch.float16:
        scaler = O.DynamicGradScalerOracle(initial_scale=256.0, min_scale=1, max_scale=2**24, hysteresis=1)
    else:    # bfloat16 trains with a constant scale of 1; the overflow check still runs
        scaler = O.ConstantGradScalerOracle(1.0)
    assert opt.gated_step and len(module.param_chunks) >= 2
    before = [(pc.paired_chunk.shard.clone(), *[t.clone() for t in opt._binding.moments(pc.paired_chunk)])
              for pc in module.param_chunks]
    for pc in module.param_chunks:
        pc.shard[pc.n_valid:] = 7.0                      # garbage in the padding
        pc.invalidate_stats()
    module.param_chunks[0].shard[11] = float('inf')
    refresh_oracle_grads(module, ochunks)
    opt.mark_gradients_scaled()
    opt.step()
    info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=1.0)
    assert opt.last_step_info['found_inf'] is True and info['found_inf'] is True
    assert opt.loss_scale == info['loss_scale'] == (128.0 if dtype == torch.float16 else 1.0)
    for pc, (p0, m0, v0) in zip(module.param_chunks, before):
        m, v = opt._binding.moments(pc.paired_chunk)
        assert torch.equal(pc.paired_chunk.shard, p0) and torch.equal(m, m0) and torch.equal(v, v0)
        assert torch.equal(pc.shard, p0.to(dtype))      # the whole shard, padding included
    assert set(st['step'] for st in opt.state.values()) == {0}
    gen = torch.Generator(device=DEV).manual_seed(52)
    for pc in module.param_chunks:
        g = torch.randn(pc.shard_size, generator=gen, device=DEV) * (2e-2 * opt.loss_scale)
        g[pc.utilized_size:] = 0
        pc.shard.copy_(g.to(dtype))
        pc.invalidate_stats()
    refresh_oracle_grads(module, ochunks)
    opt.mark_gradients_scaled()
    opt.step()
    info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=1.0)
    assert opt.last_step_info['found_inf'] is False and set(st['step'] for st in opt.state.values()) == {1}
    compare_state(module, opt, ochunks, dtype, rtol=1e-6, atol_p=1e-9, atol_m=1e-8, atol_v=1e-10, tag='after the skip')


@pytest.mark.parametrize('gated', [True, False])
def test_a_skipped_step_is_logged_where_the_reference_logs_it(oracle, caplog, gated):
    """optimizer.py:199: 'Found overflow. Skip step' at INFO, once per skipped step, on either way the step is
    decided; a step that happens logs nothing."""
    import logging
    module, opt, ochunks = build_workload([('a', (5000, )), ('b', (300, 7))], 1 << 13, torch.float16, seed=61,
                                          loss_scale=64.0, initial_scale=64.0, hysteresis=1)
    opt.gated_step = gated
    caplog.set_level(logging.INFO, logger='elixir_amd.optimizer')
    opt.mark_gradients_scaled()
    opt.step()
    assert opt.last_step_info['found_inf'] is False and not caplog.records
    module.param_chunks[0].shard[3] = float('nan')
    for pc in module.param_chunks:
        pc.invalidate_stats()
    opt.mark_gradients_scaled()
    opt.step()
    assert opt.last_step_info['found_inf'] is True
    assert [(r.name, r.levelname, r.getMessage()) for r in caplog.records] == [
        ('elixir_amd.optimizer', 'INFO', 'Found overflow. Skip step')]
