"""The step at the full sizes of the benchmark workloads (GPT-2 small, OPT-1.3B, LLaMA-7B chunk
sets).  The oracle cannot chew through billions of elements in seconds, so the checks here are the
ones that do not depend on size:

  * the update is element-wise, so ANY slice of a chunk is a complete small problem: seeded slices
    (segment heads and tails, chunk tails with padding, random interiors) are replayed by the CPU
    oracle from the pre-step state and must match the GPU's post-step state;
  * the gradient norm is additive: the global norm the step used equals the float64 sum over
    torch-computed slice norms;
  * writeback is idempotent and total: after the step every low-precision shard equals the cast of
    its master shard, padding included;
  * a skipped step (overflow) leaves master / exp_avg / exp_avg_sq bit-identical, restores the
    low-precision shards, and moves the loss scale as the state machine says;
  * the step is deterministic: replaying it from the same state gives the same bits.

The C oracle does run at about 10**9 elements a second on the box's cores, which is enough to replay
EVERY element once: ``test_full_size_every_element`` steps each set on the GPU, replays it chunk by
chunk on the CPU from a pre-step clone and compares all of master, exp_avg, exp_avg_sq and the
low-precision shard bit for bit.
"""
import math

import numpy as np
import pytest
import torch

from elixir_amd import workloads
from oracle import oracle as O

from helpers import CODE, to_np, ulp_distance

pytestmark = pytest.mark.gpu


def _slices(pc, opt, rng, width=4096, n_random=6):
    """(begin, end) windows of one chunk: around every few segment boundaries, the chunk tail
    (valid end and padding), and random interiors."""
    oc = pc.paired_chunk
    n = pc.shard_size
    bounds = sorted({b for f, c in opt.param_to_optim_chunk.items() if c is oc for b in opt.param_to_range[f]})
    picks = set()
    for b in bounds[::max(1, len(bounds) // 6)]:
        picks.add(max(0, min(n - width, b - width // 2)))
    picks.add(max(0, n - width))
    picks.add(max(0, min(n - width, pc.utilized_size - width // 2)))
    for _ in range(n_random):
        picks.add(int(rng.integers(0, max(1, n - width))))
    return [(b, min(n, b + width)) for b in sorted(picks)]


def _oracle_on_slice(pc, opt, b, e, pre, comb, dtype):
    """Replays the update on [b, e) of one chunk with the CPU oracle; returns (p, m, v, lowp)."""
    oc = pc.paired_chunk
    g, p, m, v = (a.copy() for a in pre)
    inner = opt.optim
    for group in inner.param_groups:
        for fake in group['params']:
            if opt.param_to_optim_chunk[fake] is not oc:
                continue
            sb, se = opt.param_to_range[fake]
            lo, hi = max(sb, b), min(se, e)
            if lo >= hi:
                continue
            sl = slice(lo - b, hi - b)
            O.adam(g[sl], CODE[dtype], p[sl], m[sl], v[sl], lr=group['lr'], beta1=group['betas'][0],
                   beta2=group['betas'][1], eps=group['eps'], weight_decay=group['weight_decay'],
                   step=inner.state[fake]['step'], adamw_mode=inner.adamw_mode,
                   bias_correction=group['bias_correction'], div_scale=float(comb))
    return p, m, v, O.writeback(p, CODE[dtype])


@pytest.mark.parametrize('name', ['c2', 'c4', 'c5'])
def test_full_size_step(oracle, name):
    built = workloads.build(name, seed=4321)
    opt, module, dtype = built.optimizer, built.module, built.spec.dtype
    rng = np.random.default_rng(11)
    binding = opt._binding

    # ---- a clean step, checked on slices ------------------------------------------------------
    built.land_gradients()
    windows, pre = {}, {}
    norm_sq = 0.0
    for ci, pc in enumerate(module.param_chunks):
        oc = pc.paired_chunk
        m, v = binding.moments(oc)
        windows[ci] = _slices(pc, opt, rng)
        for (b, e) in windows[ci]:
            pre[(ci, b)] = (to_np(pc.shard[b:e]), to_np(oc.shard[b:e]), to_np(m[b:e]), to_np(v[b:e]))
        if built.spec.max_norm > 0:
            # per-chunk squared norm the way the reference takes it (chunk.py:218-221), with torch
            norm_sq += float(pc.shard[:pc.n_valid].float().norm(2).item())**2
    opt.step()
    info = opt.last_step_info
    assert info['found_inf'] is False
    if built.spec.max_norm > 0:
        assert math.isclose(info['total_norm'], math.sqrt(norm_sq), rel_tol=1e-6)
        want_comb = O.combined_scale(built.spec.loss_scale, info['total_norm'], built.spec.max_norm)
        assert info['combined_scale'] == want_comb
    else:
        assert info['combined_scale'] == O.combined_scale(built.spec.loss_scale, None, 0.0)
    comb = info['combined_scale']
    assert all(st['step'] == 1 for st in opt.state.values())

    for ci, pc in enumerate(module.param_chunks):
        oc = pc.paired_chunk
        m, v = binding.moments(oc)
        for (b, e) in windows[ci]:
            wp, wm, wv, wl = _oracle_on_slice(pc, opt, b, e, pre[(ci, b)], comb, dtype)
            tag = f'{name} chunk {ci} [{b},{e})'
            assert np.array_equal(to_np(oc.shard[b:e]).view(np.uint32), wp.view(np.uint32)), tag + ' master'
            assert np.array_equal(to_np(m[b:e]).view(np.uint32), wm.view(np.uint32)), tag + ' exp_avg'
            assert np.array_equal(to_np(v[b:e]).view(np.uint32), wv.view(np.uint32)), tag + ' exp_avg_sq'
            assert ulp_distance(to_np(pc.shard[b:e]), wl) == 0, tag + ' writeback'
        # writeback is total: the whole low-precision shard is the cast of the master shard
        assert torch.equal(pc.shard, oc.shard.to(dtype)), f'{name} chunk {ci}: shard != cast(master)'
        assert pc.optim_sync_flag is True

    # ---- determinism: replay the same step from a restored slice of state ---------------------
    ci = 0
    pc = module.param_chunks[ci]
    oc = pc.paired_chunk
    m, v = binding.moments(oc)
    after = (oc.shard[:65536].clone(), m[:65536].clone(), v[:65536].clone())

    # ---- an overflow: skip, restore, back off --------------------------------------------------
    built.land_gradients()
    last = module.param_chunks[-1]
    last.shard[last.n_valid - 1] = float('nan')
    if last.n_valid < last.shard_size:
        last.shard[last.n_valid] = float('inf')           # padding: must not matter
    keep = [(pc.paired_chunk.shard[:65536].clone(), *(t[:65536].clone() for t in binding.moments(pc.paired_chunk)))
            for pc in module.param_chunks]
    scale_before = opt.loss_scale
    opt.step()
    assert opt.last_step_info['found_inf'] is True
    assert opt.loss_scale == (scale_before * 0.5 if module.use_amp else scale_before)
    assert all(st['step'] == 1 for st in opt.state.values())
    for pc, (p0, m0, v0) in zip(module.param_chunks, keep):
        oc = pc.paired_chunk
        m, v = binding.moments(oc)
        assert torch.equal(oc.shard[:65536], p0) and torch.equal(m[:65536], m0) and torch.equal(v[:65536], v0)
        assert torch.equal(pc.shard, oc.shard.to(dtype))
    assert torch.equal(after[0], oc.shard[:65536] if False else module.param_chunks[0].paired_chunk.shard[:65536])

    # ---- a clean follow-up step at the new scale passes the same slice check ------------------
    if module.use_amp:
        for pc, g in zip(module.param_chunks, built.grads):
            g.mul_(0.5)                                    # the same gradients at the halved loss scale
    built.land_gradients()
    pc = module.param_chunks[1 % len(module.param_chunks)]
    oc = pc.paired_chunk
    m, v = binding.moments(oc)
    b, e = windows[1 % len(module.param_chunks)][0]
    pre1 = (to_np(pc.shard[b:e]), to_np(oc.shard[b:e]), to_np(m[b:e]), to_np(v[b:e]))
    opt.step()
    assert opt.last_step_info['found_inf'] is False
    assert all(st['step'] == 2 for st in opt.state.values())
    wp, wm, wv, wl = _oracle_on_slice(pc, opt, b, e, pre1, opt.last_step_info['combined_scale'], dtype)
    assert np.array_equal(to_np(oc.shard[b:e]).view(np.uint32), wp.view(np.uint32))
    assert np.array_equal(to_np(m[b:e]).view(np.uint32), wm.view(np.uint32))
    assert ulp_distance(to_np(pc.shard[b:e]), wl) == 0


def _host(t: torch.Tensor) -> np.ndarray:
    """Device tensor -> numpy without a second host copy; 16-bit floats as uint16 bit patterns."""
    t = t.detach()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


@pytest.mark.parametrize('name', ['c2', 'c4', 'c5'])
def test_full_size_every_element(oracle, name):
    """Element for element at full size: the pre-step state of every chunk is cloned on the device, the
    set is stepped once on the GPU, and every chunk is then replayed on the CPU by the oracle (one
    ``adam`` call per tensor, with the combined scale the GPU's step reports, then the cast of the whole
    shard).  Identical bits for master / exp_avg / exp_avg_sq and for the low-precision shard over all
    ``shard_size`` elements of every chunk: padding refreshed, nothing outside the tensors touched."""
    import gc
    import time
    gc.collect()
    torch.cuda.empty_cache()    # what earlier tests left with the caching allocator goes back to the driver
    built = workloads.build(name, seed=2468)
    opt, module, dtype = built.optimizer, built.module, built.spec.dtype
    code = CODE[dtype]
    binding, inner = opt._binding, opt.optim
    built.land_gradients()
    need = 12 * built.n_alloc
    free, _ = torch.cuda.mem_get_info()
    free += torch.cuda.memory_reserved() - torch.cuda.memory_allocated()
    assert free > need + (4 << 30), f'{name}: {free >> 30} GiB free, the pre-step clone needs {need >> 30} GiB'
    pre = []
    for pc in module.param_chunks:
        oc = pc.paired_chunk
        m, v = binding.moments(oc)
        pre.append((oc.shard.clone(), m.clone(), v.clone()))    # the gradients are built.grads
    opt.step()
    info = opt.last_step_info
    assert info['found_inf'] is False
    comb = float(info['combined_scale'])
    if built.spec.max_norm > 0:
        assert comb > built.spec.loss_scale    # the clip is active: a divisor that is not a power of two
    torch.cuda.synchronize()

    t0 = time.perf_counter()
    checked = 0
    for ci, pc in enumerate(module.param_chunks):
        oc = pc.paired_chunk
        gm, gv = binding.moments(oc)
        p0, m0, v0 = pre[ci]
        pn, mn, vn, gn = _host(p0), _host(m0), _host(v0), _host(built.grads[ci])
        pre[ci] = None
        del p0, m0, v0
        covered = 0
        for group in inner.param_groups:
            for fake in group['params']:
                if opt.param_to_optim_chunk[fake] is not oc:
                    continue
                b, e = opt.param_to_range[fake]
                assert inner.state[fake]['step'] == 1
                oracle.adam(gn[b:e], code, pn[b:e], mn[b:e], vn[b:e], lr=group['lr'], beta1=group['betas'][0],
                            beta2=group['betas'][1], eps=group['eps'], weight_decay=group['weight_decay'], step=1,
                            adamw_mode=inner.adamw_mode, bias_correction=group['bias_correction'], div_scale=comb)
                covered += e - b
        assert covered == pc.utilized_size
        tag = f'{name} chunk {ci}'
        assert np.array_equal(_host(oc.shard).view(np.uint32), pn.view(np.uint32)), tag + ' master'
        assert np.array_equal(_host(gm).view(np.uint32), mn.view(np.uint32)), tag + ' exp_avg'
        assert np.array_equal(_host(gv).view(np.uint32), vn.view(np.uint32)), tag + ' exp_avg_sq'
        assert np.array_equal(_host(pc.shard), oracle.writeback(pn, code)), tag + ' low-precision shard'
        if pc.utilized_size < pc.shard_size:    # the padding: zero master, never updated, refreshed to zero
            assert not pn[pc.utilized_size:].any() and not mn[pc.utilized_size:].any()
        checked += pc.shard_size
        print(f'{tag}: {pc.shard_size} elements identical ({time.perf_counter() - t0:.1f} s)', flush=True)
    assert checked == built.n_alloc


def test_full_size_step_is_deterministic():
    a = workloads.build('c2', seed=99)
    a.land_gradients()
    a.optimizer.step()
    first = [(pc.paired_chunk.shard.clone(), pc.shard.clone()) for pc in a.module.param_chunks]
    norm = a.optimizer.last_step_info
    del a
    b = workloads.build('c2', seed=99)
    b.land_gradients()
    b.optimizer.step()
    assert b.optimizer.last_step_info == norm
    for (p0, l0), pc in zip(first, b.module.param_chunks):
        assert torch.equal(p0, pc.paired_chunk.shard) and torch.equal(l0, pc.shard)


def test_one_buffer_beyond_two_to_the_32_elements():
    """Element offsets are 64-bit everywhere: one flat fp32 parameter of 2**32 + 2**20 + 77 elements
    with fp16 gradients goes through the update, the single-buffer stats and the single-buffer
    refresh; windows at the start, across the 2**32 boundary and at the ragged end are replayed by
    the oracle, and a non-finite value planted behind the boundary is found."""
    import elixir_amd as ea
    from elixir_amd import _abi
    dev = 'cuda'
    n = (1 << 32) + (1 << 20) + 77
    gen = torch.Generator(device=dev).manual_seed(5)
    p = torch.nn.Parameter(torch.empty(n, device=dev))
    p.data.normal_(0, 0.02, generator=gen)
    g = torch.empty(n, dtype=torch.float16, device=dev)
    g.normal_(0, 0.5, generator=gen)
    windows = [(0, 5000), ((1 << 32) - 3001, (1 << 32) + 2999), (n - 4000, n)]
    pre = [(to_np(g[b:e]).copy(), to_np(p.data[b:e]).copy()) for b, e in windows]
    opt = ea.HybridAdam([p], lr=1e-2, weight_decay=0.1)
    p.grad_dtype = None
    p.grad = g
    opt.step(div_scale=48.0)
    st = opt.state[p]
    for (b, e), (gn, pn) in zip(windows, pre):
        mn, vn = np.zeros(e - b, np.float32), np.zeros(e - b, np.float32)
        O.adam(gn, O.F16, pn, mn, vn, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.1, step=1,
               adamw_mode=True, div_scale=48.0)
        for name, got, want in (('p', p.data, pn), ('m', st['exp_avg'], mn), ('v', st['exp_avg_sq'], vn)):
            assert np.array_equal(to_np(got[b:e]).view(np.uint32), want.view(np.uint32)), (name, b, e)
    # every element was updated exactly once: exp_avg = 0.1 * g / 48 everywhere
    assert torch.equal(st['exp_avg'][::4099] != 0, g[::4099] != 0)
    del st, opt
    # single-buffer stats over the whole run, clean and with a NaN behind the 2**32 boundary
    stream = torch.cuda.current_stream().cuda_stream
    blocks = 1024
    ws = torch.empty((blocks + 1) * 16, dtype=torch.uint8, device=dev)

    def stats():
        _abi.grad_stats(g.data_ptr(), O.F16, n, blocks, ws.data_ptr(), ws.data_ptr() + blocks * 16, stream)
        return ws[blocks * 16:].cpu().numpy().view(_abi.STATS_DTYPE)[0]

    rec = stats()
    ref = sum(float(g[i:i + (1 << 28)].double().square().sum()) for i in range(0, n, 1 << 28))
    assert rec['overflow'] == 0 and abs(float(rec['sumsq']) - ref) <= 1e-6 * ref
    g[(1 << 32) + 12345] = float('nan')
    assert stats()['overflow'] == 1
    g[(1 << 32) + 12345] = 0.0
    g[n - 1] = float('inf')
    assert stats()['overflow'] == 1
    # single-buffer refresh: the whole run, checked in the same windows
    low = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    _abi.writeback(p.data.data_ptr(), low.data_ptr(), O.BF16, n, stream)
    for b, e in windows:
        assert torch.equal(low[b:e], p.data[b:e].to(torch.bfloat16)), (b, e)
    assert int(torch.count_nonzero(low[::4099])) == int(torch.count_nonzero(p.data[::4099].to(torch.bfloat16)))


def test_one_table_row_beyond_two_to_the_32_elements():
    """The table forms over ONE row of 2**32 + 2**20 + 77 elements, straight through the C ABI: the landing
    launch (every element moved by workgroups that take several tiles each, the flags of the valid head
    taken, a non-finite value behind the 2**32 boundary found, one in the padding ignored), the stats launch
    over the same row, and the refresh launch (several pieces per workgroup)."""
    from elixir_amd import _abi
    from elixir_amd.chunk import DeviceTable
    dev = torch.device('cuda', 0)
    stream = torch.cuda.current_stream().cuda_stream
    n = (1 << 32) + (1 << 20) + 77
    n_valid = n - 1000
    step = 1 << 28
    gen = torch.Generator(device=dev).manual_seed(6)
    src = torch.empty(n, dtype=torch.float16, device=dev)
    src.normal_(0, 0.5, generator=gen)
    dst = torch.empty(n, dtype=torch.float16, device=dev)
    dst.fill_(7.0)
    rows = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
    rows[0]['grad'], rows[0]['lowp_out'], rows[0]['n_alloc'], rows[0]['n_valid'] = src.data_ptr(), dst.data_ptr(), n, n_valid
    table = DeviceTable(rows, dev)
    bpr = _abi.check_land_rows(rows, None, O.F16, O.F16)
    assert bpr == _abi.land_max_blocks() < -(-n // _abi.land_tile_elems(O.F16))    # more tiles than workgroups
    ws = torch.empty(_abi.land_workspace_records(1, bpr, 1) * 16, dtype=torch.uint8, device=dev)
    out = torch.zeros(16, dtype=torch.uint8, device=dev)

    def land():
        _abi.land_grads_mt(table.ptr, 1, O.F16, O.F16, 1.0, bpr, ws.data_ptr(), out.data_ptr(), True, stream)
        return out.cpu().numpy().view(_abi.STATS_DTYPE)[0]

    def same(a, b):
        return all(torch.equal(a[i:i + step].view(torch.int16), b[i:i + step].view(torch.int16)) for i in range(0, n, step))

    rec = land()
    assert same(dst, src)
    ref = sum(float(src[i:min(n_valid, i + step)].double().square().sum()) for i in range(0, n_valid, step))
    # (against the exact sum both launches sit 5e-8 low, alike: the square of a 16-bit value m * 2**e has
    # m * m mod 4 in {0, 1}, so the bits an fp32 partial sum rounds away are below one half more often than above)
    assert rec['overflow'] == 0 and abs(float(rec['sumsq']) - ref) <= 1e-6 * ref

    # the stats launch over the same row: the same flags, the same sum to the last few bits
    stats_rows = rows.copy()
    stats_rows[0]['grad'], stats_rows[0]['lowp_out'] = dst.data_ptr(), 0
    stats_table = DeviceTable(stats_rows, dev)
    partials = torch.empty(1024 * 16, dtype=torch.uint8, device=dev)
    out2 = torch.zeros(16, dtype=torch.uint8, device=dev)

    def stats():
        _abi.grad_stats_mt(stats_table.ptr, 1, O.F16, 1024, partials.data_ptr(), out2.data_ptr(), False, stream)
        return out2.cpu().numpy().view(_abi.STATS_DTYPE)[0]

    rec2 = stats()
    assert rec2['overflow'] == 0 and abs(float(rec2["sumsq"]) - float(rec["sumsq"])) <= 1e-9 * ref

    src[n_valid + 5] = float('inf')                       # in the padding: moved, not counted
    rec = land()
    assert rec['overflow'] == 0 and same(dst, src) and stats()['overflow'] == 0
    src[(1 << 32) + 999] = float('nan')                   # behind the boundary, inside the valid head
    assert land()['overflow'] == 1 and stats()['overflow'] == 1
    src[(1 << 32) + 999] = 0.0
    src[n_valid - 1] = float('-inf')                      # the last valid element
    assert land()['overflow'] == 1 and stats()['overflow'] == 1
    del src, ws, partials

    # the refresh launch over one row: fp32 master -> bf16, 4.2 M pieces over at most 2**20 workgroups
    master = torch.empty(n, dtype=torch.float32, device=dev)
    master.normal_(0, 0.02, generator=gen)
    low = dst.view(torch.bfloat16)
    low.fill_(7.0)
    wb_rows = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
    wb_rows[0]['lowp_out'], wb_rows[0]['master'], wb_rows[0]['n_alloc'] = low.data_ptr(), master.data_ptr(), n
    wb_table = DeviceTable(wb_rows, dev)
    assert -(-n // _abi.refresh_piece_elems()) > 1 << 20
    _abi.writeback_mt(wb_table.ptr, 1, O.BF16, n, True, stream)
    for i in range(0, n, step):
        assert torch.equal(low[i:i + step], master[i:i + step].to(torch.bfloat16)), i


def test_one_chunk_beyond_two_to_the_32_elements_through_the_optimizer(oracle):
    """A chunk of 2**32 + 2**25 elements in which one tensor crosses element 2**32, through ElixirOptimizer
    (clipped AdamW, fp16 x 2**16): stepped once with its own stats pass and once behind a fused landing;
    windows at the segment boundaries, across elements 2**31 and 2**32 and at the ragged end are replayed by
    the oracle, the norm is held against torch's, the whole low-precision shard equals the cast of the
    master shard, and an inf planted behind element 2**32 skips the step."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    shapes = [('a.weight', (3000, 4096)), ('big.weight', ((1 << 32) + 4096, )), ('b.bias', (2 << 19, )), ('c.weight', (77, 8))]
    built = workloads.build('c5', shapes=shapes, chunk_size=(1 << 32) + (1 << 25), seed=9)
    opt, module, dtype = built.optimizer, built.module, built.spec.dtype
    assert len(module.param_chunks) == 1 and built.n_valid == sum(int(np.prod(s)) for _, s in shapes) > 1 << 32
    pc = module.param_chunks[0]
    oc = pc.paired_chunk
    m, v = opt._binding.moments(oc)
    rng = np.random.default_rng(1)
    piece = 1 << 28
    for fused in (False, True):
        built.land_gradients(fused=fused)
        wins = _slices(pc, opt, rng) + [((1 << 32) - 2048, (1 << 32) + 2048), ((1 << 31) - 100, (1 << 31) + 100)]
        pre = {b: (to_np(pc.shard[b:e]), to_np(oc.shard[b:e]), to_np(m[b:e]), to_np(v[b:e])) for b, e in wins}
        norm_sq = sum(float(pc.shard[i:min(pc.n_valid, i + piece)].float().norm(2).item())**2 for i in range(0, pc.n_valid, piece))
        opt.step()
        info = opt.last_step_info
        assert info['found_inf'] is False and math.isclose(info['total_norm'], math.sqrt(norm_sq), rel_tol=1e-6)
        assert info['combined_scale'] == O.combined_scale(built.spec.loss_scale, info['total_norm'], built.spec.max_norm)
        for b, e in wins:
            wp, wm, wv, wl = _oracle_on_slice(pc, opt, b, e, pre[b], info['combined_scale'], dtype)
            assert np.array_equal(to_np(oc.shard[b:e]).view(np.uint32), wp.view(np.uint32)), (fused, b, e)
            assert np.array_equal(to_np(m[b:e]).view(np.uint32), wm.view(np.uint32)), (fused, b, e)
            assert np.array_equal(to_np(v[b:e]).view(np.uint32), wv.view(np.uint32)), (fused, b, e)
            assert ulp_distance(to_np(pc.shard[b:e]), wl) == 0, (fused, b, e)
        for i in range(0, pc.shard_size, piece):
            assert torch.equal(pc.shard[i:i + piece], oc.shard[i:i + piece].to(dtype)), (fused, i)
    keep = (oc.shard[(1 << 32):(1 << 32) + 65536].clone(), m[(1 << 32):(1 << 32) + 65536].clone())
    built.land_gradients(fused=True)
    pc.shard[(1 << 32) + 5000] = float('inf')
    pc.invalidate_stats()
    opt.mark_gradients_scaled()
    scale = opt.loss_scale
    opt.step()
    assert opt.last_step_info['found_inf'] is True and opt.loss_scale == scale * 0.5
    assert torch.equal(keep[0], oc.shard[(1 << 32):(1 << 32) + 65536]) and torch.equal(keep[1], m[(1 << 32):(1 << 32) + 65536])
    for i in range(0, pc.shard_size, piece):
        assert torch.equal(pc.shard[i:i + piece], oc.shard[i:i + piece].to(dtype)), i
