#!/usr/bin/env python3
"""Benchmark of the optimizer step (ElixirOptimizer.step over chunk-packed parameters) on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c4|c2|c1|velocity] [--no-configs]

A step is one full pass of the hot path over one set of synthetic gradients that already sit in
the low-precision chunk shards: stats launch (overflow flag + sum of squares) -> fold + decision
kernel (skip, global norm, combined scale) -> fused unscale + AdamW + low-precision writeback launch
-> refresh of the padding; the decision and the flags reach the host through pinned memory for its
bookkeeping while the update runs.  Step time is host wall-clock between two device
synchronisations, so host overhead counts.  Prints ONE JSON line: the headline workload (c5 unless
--workload says otherwise) and, on the default run, a `configs` object with the other configurations
(c1, c2, c4 and the reference's own flat-parameter micro-benchmark) measured the same way.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X published HBM3E bandwidth
BYTES_UPDATE = 28               # per valid element: read g(2)+p,m,v(12); write p,m,v(12)+lowp(2)
BYTES_STATS = 2                 # per valid element: the compulsory second read of g
# HBM bytes per adam_step_kernel launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script, scaled by what the same counters read for a plain copy of known size (--calibrate-copy).
# Counter runs cannot ride along with a timed run, so the figure is a recorded one: it is only put into
# the line while the device code is still the one it was measured on (sha256 over elx_kernels.hip and
# elx_host.h, first 16 hex digits), and the line names the summary it comes from.
RECORDED_TRAFFIC = {
    # workload: (bytes per launch, summary under profiles/, kernel source the counters were read on)
    'c5': (94.411e9 + 94.364e9, 'profiles/adam_step_kernel_c5_llama7b.md', 'ee4bbd5dc2fdbf61'),
    'c4': (18.4445e9 + 18.4305e9, 'profiles/all_kernels_c4_opt1b3_c2_gpt2_c1.md', 'ee4bbd5dc2fdbf61'),
}
DEVICE_SOURCES = [os.path.join(ROOT, 'elixir_amd', 'csrc', name) for name in ('elx_kernels.hip', 'elx_host.h')]


def kernel_source_sha16() -> str:
    """Digest of the files the device code is made from (the kernels and the header with the constants that
    shape them); the recorded counter figures name the digest they were read on."""
    import hashlib
    h = hashlib.sha256()
    for path in DEVICE_SOURCES:
        with open(path, 'rb') as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def traffic_fields(workload: str):
    """(traffic, traffic_source) of the roofline object: the recorded counter figure when it was read on
    the kernel source that is built now, else None with the reason."""
    rec = RECORDED_TRAFFIC.get(workload)
    if rec is None:
        return None, None
    nbytes, summary, sha = rec
    now = kernel_source_sha16()
    if sha != now:
        return None, {'summary': summary, 'note': f'counters were read on kernel source {sha}, this build is {now}: stale'}
    from elixir_amd import _abi
    return nbytes, {'summary': summary, 'kernel_source_sha16': sha,
                    # _abi.load() has refused a library that was not built from the sources beside it
                    'library_built_from': (_abi.load().elx_source_sha() or b'').decode(),
                    'method': 'rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by a plain copy of known size'}


def cpu_baseline(built, sample_elems: int, steps: int = 8):
    """The same step as torch CPU ops (the oracle's torch harness) on a bounded sample: the first
    `sample_elems` elements of chunk 0.  Returns the cpu_baseline object of the JSON line."""
    from oracle import oracle as O
    from oracle.torch_ref import TorchCpuStep
    spec = built.spec
    pc = built.module.param_chunks[0]
    oc = pc.paired_chunk
    n = min(sample_elems, pc.utilized_size)
    m, v = built.optimizer._binding.moments(oc)
    master = oc.shard[:n].cpu()
    g = built.grads[0][:n].cpu()
    ref = TorchCpuStep(master, spec.dtype, lr=spec.lr, betas=spec.betas, eps=spec.eps, weight_decay=spec.weight_decay,
                       adamw_mode=spec.adamw_mode, exp_avg=m[:n].cpu(), exp_avg_sq=v[:n].cpu())
    times = []
    for i in range(steps + 1):
        t0 = time.perf_counter()
        ref.step(g, loss_scale=spec.loss_scale, max_norm=spec.max_norm)
        times.append(time.perf_counter() - t0)
    t = float(np.median(times[1:]))

    # the C restatement (OpenMP) on the same sample, for reference
    code = {torch.float16: O.F16, torch.bfloat16: O.BF16, torch.float32: O.F32}[spec.dtype]
    gb = g.view(torch.int16).numpy().view(np.uint16).copy() if code != O.F32 else g.numpy().copy()
    pn, mn, vn = master.numpy().copy(), m[:n].cpu().numpy().copy(), v[:n].cpu().numpy().copy()
    ctimes = []
    for i in range(steps + 1):
        t0 = time.perf_counter()
        O.overflow(gb, code)
        O.l2norm_sq_ref(gb, code)
        O.adam(gb, code, pn, mn, vn, lr=spec.lr, beta1=spec.betas[0], beta2=spec.betas[1], eps=spec.eps,
               weight_decay=spec.weight_decay, step=i + 1, adamw_mode=spec.adamw_mode, div_scale=spec.loss_scale * 1.5)
        O.writeback(pn, code)
        ctimes.append(time.perf_counter() - t0)
    tc = float(np.median(ctimes[1:]))
    return {
        'value': n / t,
        'unit': 'elements/s',
        'cores': torch.get_num_threads(),
        'kind': 'port',
        'sample': f'first {n} elements of chunk 0 of {spec.name}; torch CPU ops (isinf/isnan, float().norm, '
                  f'float().div_, torch.optim.AdamW, .to(lowp)); median of {steps} steps after 1 warm-up',
        'extrapolation': f'per-element rate of the sample, linear: the whole set of {built.n_valid} elements at this '
                         f'rate takes {built.n_valid / (n / t):.1f} s per step',
        'ms_per_step_sample': t * 1e3,
        'gbps_30B': 30 * n / t / 1e9,
        'oracle_c_openmp': {'value': n / tc, 'unit': 'elements/s', 'cores': O.num_threads()},
    }


def cpu_baseline_whole_set(built, steps: int = 5):
    """The torch CPU step of ``cpu_baseline`` over EVERY chunk of the set, one chunk after the other (for a set
    small enough to do so: the GPT-2 one).  No extrapolation: the time of a step is the sum over the chunks."""
    from oracle.torch_ref import TorchCpuStep
    spec = built.spec
    assert spec.max_norm == 0.0, 'a clipped step needs the global norm first; this helper times unclipped sets'
    total = 0.0
    for pc, g_dev in zip(built.module.param_chunks, built.grads):
        oc = pc.paired_chunk
        n = pc.utilized_size
        m, v = built.optimizer._binding.moments(oc)
        ref = TorchCpuStep(oc.shard[:n].cpu(), spec.dtype, lr=spec.lr, betas=spec.betas, eps=spec.eps,
                           weight_decay=spec.weight_decay, adamw_mode=spec.adamw_mode, exp_avg=m[:n].cpu(),
                           exp_avg_sq=v[:n].cpu())
        g = g_dev[:n].cpu()
        times = []
        for _ in range(steps + 1):
            t0 = time.perf_counter()
            ref.step(g, loss_scale=spec.loss_scale, max_norm=0.0)
            times.append(time.perf_counter() - t0)
        total += float(np.median(times[1:]))
        del ref, g
    return {
        'value': built.n_valid / total, 'unit': 'elements/s', 'cores': torch.get_num_threads(), 'kind': 'port',
        'sample': f'the whole configuration, {len(built.grads)} chunks one after the other: torch CPU ops (isinf/isnan, '
                  f'float().div_, torch.optim.Adam, .to(lowp)); per chunk the median of {steps} steps after 1 warm-up',
        'extrapolation': 'none: full size', 'ms_per_step_sample': total * 1e3,
    }


def fused_landing_leg(built, steps):
    """The same step when the gradients arrive through the landing launch that leaves the flags on
    the device: the step then holds no pass over the gradients (28 B per valid element).  Reports
    the landing launch itself next to the plain device copy it replaces (both outside the step)."""
    opt = built.optimizer
    chunks = built.module.param_chunks
    n_alloc, n_valid = built.n_alloc, built.n_valid
    esize = built.grads[0].element_size()

    blocker = torch.empty(2, 1 << 32, dtype=torch.uint8, device=chunks[0].shard_device)

    def behind_blocker(fn):
        """Device time of what ``fn`` enqueues: a 4 GiB copy runs in front (1.4 ms), so that the host's part of
        ``fn`` (building tables, issuing one launch per chunk) is over before the device gets to its launches."""
        b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        blocker[1].copy_(blocker[0])
        b.record()
        fn()
        e.record()
        e.synchronize()
        return b.elapsed_time(e) * 1e-3

    def plain():
        for pc, g in zip(chunks, built.grads):
            pc.shard.copy_(g)

    plain_s, land_s, step_s = [], [], []
    for i in range(steps + 1):
        t_plain = behind_blocker(plain)
        for pc in chunks:
            pc.invalidate_stats()
        t_land = behind_blocker(lambda: built.land_gradients(fused=True))
        torch.cuda.synchronize()
        # the flags of every chunk wait in the device arena: the step launches no pass over the gradients
        assert opt._stats_source()[0] == 'arena'
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert opt.last_step_info['found_inf'] is False
        if i > 0:
            plain_s.append(t_plain)
            land_s.append(t_land)
            step_s.append(dt)
    t_step, t_land, t_plain = float(np.mean(step_s)), float(np.mean(land_s)), float(np.mean(plain_s))

    # the flow of a training loop: backward lands every chunk with a launch of its own as soon as its last
    # gradient exists, the last chunk first; the records still end up side by side (the optimizer gave every
    # chunk its slot in chunk order) and the step is decided on the device
    from elixir_amd.chunk import land_chunks, land_tensors
    grads = {}    # views of the saved buffers stand in for the .grad tensors
    for pc, g in zip(chunks, built.grads):
        for t, info in pc.tensors_info.items():
            grads[t] = g[info.offset:info.end]
    pc_land_s, pc_step_s, pc_payload_s = [], [], []
    for i in range(steps + 1):
        for pc in chunks:
            pc.invalidate_stats()

        def payload_by_payload():
            for pc, g in zip(reversed(chunks), reversed(built.grads)):
                land_chunks([pc], [g])

        def one_by_one():    # what ElixirModule's gradient hook issues: a chunk's own per-tensor gradients, one launch
            for pc in reversed(chunks):
                land_tensors([pc], lambda t: grads[t])

        t_pc_payload = behind_blocker(payload_by_payload)
        for pc in chunks:
            pc.invalidate_stats()
        t_pc_land = behind_blocker(one_by_one)
        opt.mark_gradients_scaled()
        torch.cuda.synchronize()
        assert opt._stats_source()[0] == 'arena'
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert opt.last_step_info['found_inf'] is False
        if i > 0:
            pc_land_s.append(t_pc_land)
            pc_payload_s.append(t_pc_payload)
            pc_step_s.append(dt)
    t_pc_step, t_pc_land = float(np.mean(pc_step_s)), float(np.mean(pc_land_s))

    # the same landing straight from per-tensor gradients (views of the saved buffers stand in for
    # the .grad tensors), next to what it replaces: a zeroed payload per chunk, one slice copy per
    # tensor, and the copy of the payload into the shard
    def slice_copies():
        for pc in chunks:
            payload = torch.zeros(pc.chunk_size, dtype=pc.chunk_dtype, device=pc.shard_device)
            for t, info in pc.tensors_info.items():
                payload[info.offset:info.end].copy_(grads[t])
            pc.shard.copy_(payload)

    pt_gpu, pt_wall, sc_gpu = [], [], []
    for i in range(steps + 1):
        a = behind_blocker(slice_copies)
        for pc in chunks:
            pc.invalidate_stats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        land_tensors(chunks, lambda t: grads[t])
        torch.cuda.synchronize()
        w = time.perf_counter() - t0
        for pc in chunks:
            pc.invalidate_stats()
        b = behind_blocker(lambda: land_tensors(chunks, lambda t: grads[t]))
        if i > 0:
            sc_gpu.append(a)
            pt_gpu.append(b)
            pt_wall.append(w)
    del blocker
    assert not any(pc.overflow for pc in chunks)
    return {
        'what': 'gradients landed by land_grads_kernel (copy + flags in one pass, outside the step); '
                'the step fetches the flags and runs the update',
        'steps': steps,
        'ms_per_step': t_step * 1e3,
        'elements_per_sec': n_valid / t_step,
        'step_gbps_28B': BYTES_UPDATE * n_valid / t_step / 1e9,
        'step_frac_28B': BYTES_UPDATE * n_valid / t_step / 1e9 / HBM_PEAK_GBPS,
        'per_chunk_landing': {
            'what': 'every chunk landed by a launch of its own straight from its per-tensor gradients, the last chunk '
                    'first (what the hooks of backward do); the step that follows is decided on the device all the same',
            'launches': len(chunks),
            'landing_ms_all_chunks': t_pc_land * 1e3,
            'landing_ms_all_chunks_from_payloads': float(np.mean(pc_payload_s)) * 1e3,
            'ms_per_step': t_pc_step * 1e3,
            'step_frac_28B': BYTES_UPDATE * n_valid / t_pc_step / 1e9 / HBM_PEAK_GBPS,
        },
        'land_kernel': {
            'kernel': 'land_grads_kernel+stats_fold_kernel+stats_finish_kernel',
            'ms_per_launch': t_land * 1e3,
            'bytes_per_launch': 2 * esize * n_alloc,
            'achieved': 2 * esize * n_alloc / t_land / 1e9,
            'unit': 'GB/s',
            'frac': 2 * esize * n_alloc / t_land / 1e9 / HBM_PEAK_GBPS,
            'plain_copy_ms': t_plain * 1e3,
        },
        'per_tensor_landing': {
            'what': 'the same launch fed by one row list over the %d per-tensor gradients (no payload)' % len(grads),
            'ms_on_device': float(np.mean(pt_gpu)) * 1e3,
            'ms_min_on_device': float(np.min(pt_gpu)) * 1e3,
            'frac_of_hbm_peak': 2 * esize * n_alloc / float(np.mean(pt_gpu)) / 1e9 / HBM_PEAK_GBPS,
            'vs_payload_landing': float(np.mean(pt_gpu)) / t_land,
            'ms_wall_with_table_build': float(np.mean(pt_wall)) * 1e3,
            'zero_payload_slice_copies_and_shard_copy_ms': float(np.mean(sc_gpu)) * 1e3,
        },
    }


def offload_gather_leg(mi_elements):
    """Source copy of the gather for ONE host-resident chunk of ``mi_elements`` Mi elements whose
    refresh was deferred: the cast kernel reading the pinned fp32 shard in place, against the staged
    form (fp32 shard to the GPU, then a cast copy).  Bound by the host link, not by HBM."""
    import elixir_amd as ea
    n = mi_elements << 20
    p = ea.Chunk(None, n, torch.float16, None, shard_device='cpu', temp_device='cpu', cpu_pin_memory=True)
    o = ea.Chunk(None, n, torch.float32, None, shard_device='cpu', temp_device='cpu', cpu_pin_memory=True)
    t = torch.empty(n, dtype=torch.float32).normal_(0, 0.02)
    p.append_tensor(t.half())
    o.append_tensor(t)
    p.close_chunk()
    o.close_chunk()
    p.init_pair(o)
    block = torch.empty(n, dtype=torch.float16, device='cuda')

    def timed(fn):
        b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        b.record()
        fn()
        e.record()
        e.synchronize()
        return b.elapsed_time(e) * 1e-3

    def fused():
        p.optim_sync_flag = False
        p.replicate(block)

    def staged():
        block.copy_(o.shard.to('cuda', non_blocking=True))

    fused_s = [timed(fused) for _ in range(4)][1:]
    ok = torch.equal(block.cpu(), o.shard.half())
    staged_s = [timed(staged) for _ in range(4)][1:]
    return {
        'what': 'gather source copy of one host-resident chunk, deferred refresh fused in',
        'elements': n,
        'fused_ms': float(np.mean(fused_s)) * 1e3,
        'fused_host_link_gbps': 4 * n / float(np.mean(fused_s)) / 1e9,
        'staged_ms': float(np.mean(staged_s)) * 1e3,
        'staged_extra_device_bytes': 4 * n,
        'matches_cast_of_master': bool(ok),
    }


def offload_step_leg(mi_elements, steps=5):
    """The optimizer step over ONE host-resident chunk pair (fp16 shard, fp32 master, moments, all in
    pinned host memory): the same launches read and write host memory in place, so the step is
    bound by the host link (16 B in, 14 B out per element).  Next to it, torch's CPU ops on the
    same data on this box's cores -- what a CPU Adam for offloaded shards costs."""
    import elixir_amd as ea
    from oracle.torch_ref import TorchCpuStep
    n = mi_elements << 20
    sr = ea.greedy_search([('w.weight', n)], n, torch.float16, shard_device=torch.device('cpu'))
    sr.param_chunk_plans[0].kwargs['cpu_pin_memory'] = True
    module = ea.ElixirModule({'w.weight': (n,)}, sr, dtype=torch.float16)
    inner = ea.HybridAdam(list(module.parameters()), lr=1e-3, weight_decay=0.1)
    opt = ea.ElixirOptimizer(module, inner, initial_scale=1024.0, hysteresis=1, max_norm=1.0)
    pc = module.param_chunks[0]
    oc = pc.paired_chunk
    m, v = opt._binding.moments(oc)
    oc.shard.normal_(0, 0.02)
    m.normal_(0, 1e-4)
    v.uniform_(0, 1e-6)
    g = (torch.empty(n).normal_(0, 1e-3 * 1024.0)).half()
    ref = TorchCpuStep(oc.shard.clone(), torch.float16, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.1,
                       adamw_mode=True, exp_avg=m.clone(), exp_avg_sq=v.clone())
    cpu_s = []
    for _ in range(3):
        t0 = time.perf_counter()
        ref.step(g, loss_scale=1024.0, max_norm=1.0)
        cpu_s.append(time.perf_counter() - t0)
    out = {}
    for bpc in (0, 32):
        opt.optim.blocks_per_cu = bpc
        ts = []
        for i in range(steps + 1):
            pc.shard.copy_(g)
            pc.invalidate_stats()
            opt.mark_gradients_scaled()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            opt.step()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
            assert opt.last_step_info['found_inf'] is False
        t = float(np.mean(ts[1:]))
        out['blocks_per_cu_%d' % (bpc or 13)] = {'ms_per_step': t * 1e3, 'elements_per_sec': n / t,
                                                  'host_link_gbps_30B': 30 * n / t / 1e9}
    tc = float(np.median(cpu_s[1:]))
    out.update({'what': 'optimizer step over one host-resident (pinned) chunk pair, in place over the host link',
                'elements': n,
                'torch_cpu_same_box': {'ms_per_step': tc * 1e3, 'elements_per_sec': n / tc,
                                       'cores': torch.get_num_threads()}})
    return out


def launch_sync_floor_us(samples: int = 200) -> float:
    """What the machine charges for ANY step, however short its kernel: one launch of a single wavefront
    that writes 48 bytes (elx_put_hypers with one record) between two device synchronisations; the median
    over ``samples`` in microseconds.  Launch latency on the way in, completion signal and wake-up on the
    way out."""
    from elixir_amd import _abi
    from elixir_amd.hybrid_adam import make_hyper_record
    lib = _abi.load()
    rec = make_hyper_record(1e-3, 0.9, 0.999, 1e-8, 0.0, 1, True, True)
    src = rec.ctypes.data
    dst = torch.zeros(64, dtype=torch.uint8, device='cuda')
    d_ptr = dst.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    ts = []
    for i in range(samples + 20):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        lib.elx_put_hypers(src, 1, d_ptr, stream)
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts[20:])) * 1e6


def config1_line(args, with_cpu: bool = True):
    """Configuration 1: plain fp32 Adam on one flat buffer of 16,777,216 elements (p ~ N(0, 0.02),
    g ~ N(0, 1e-2), m = v = 0 at the start, lr 1e-3, betas (0.9, 0.999), eps 1e-8, no weight decay,
    no loss scale, no stats pass, no low-precision copy) -- the case torch.optim.Adam runs on the
    CPU.  28 B per element: read p, g, m, v, write p, m, v.  The whole state (256 MiB) is exactly the
    size of the memory-side cache and the launch keeps it there between steps (ELX_FLAG_KEEP_STATE_CACHED).
    The line's own figure is the step a training loop sees: behind a 1 GiB device copy that empties that
    cache, as a forward and backward pass would (`value`, `ms_per_step`, `roofline`); the step that finds
    its state still in the cache, and steps queued back to back, stand beside it.  The timed steps carry no
    event records; the launch itself is timed in extra steps afterwards."""
    import elixir_amd as ea
    n = 1 << 24
    gen = torch.Generator(device='cuda')
    gen.manual_seed(1234 + 1)
    p = torch.nn.Parameter(torch.randn(n, device='cuda', generator=gen) * 0.02)
    g = torch.randn(n, device='cuda', generator=gen) * 1e-2
    opt = ea.HybridAdam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    p.grad = g
    junk = torch.empty(2, 256 << 20, dtype=torch.float32, device='cuda')
    extra = 6

    def timed_steps(cold: bool):
        step_s, call_s, adam_ms = [], [], []
        for i in range(args.warmup + args.steps + extra):
            if i == args.warmup + args.steps:
                opt.kernel_events = {}
            if cold:
                junk[1].copy_(junk[0])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            opt.step()
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            if args.warmup <= i < args.warmup + args.steps:
                step_s.append(dt)
                call_s.append(t1 - t0)
            elif i > args.warmup + args.steps:    # the first instrumented step creates the event pair
                ev = opt.kernel_events['adam_step']
                adam_ms.append(ev[0].elapsed_time(ev[1]))
        opt.kernel_events = None
        return step_s, call_s, float(np.mean(adam_ms)) * 1e-3

    warm_s, warm_call_s, t_upd_warm = timed_steps(cold=False)
    cold_s, cold_call_s, t_upd_cold = timed_steps(cold=True)
    # K steps in one bracket: nothing has to happen between two steps of this configuration (the gradient
    # stays where it is), so the launches can queue up behind each other and the host's share disappears
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        opt.step()
    torch.cuda.synchronize()
    t_queued = (time.perf_counter() - t0) / args.steps
    del junk
    floor_us = launch_sync_floor_us()
    t_cold, t_warm = float(np.mean(cold_s)), float(np.mean(warm_s))
    host_us = float(np.median(cold_call_s)) * 1e6
    out = {
        'metric': 'adam_elements_per_sec', 'value': n / t_cold, 'unit': 'elements/s', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': t_cold * 1e3, 'higher_is_better': True, 'scaling': 'weak',
        'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'c1: plain fp32 Adam, one flat buffer of 16Mi elements, no loss scale, no low-precision '
                               'copy; every step behind a 1 GiB device copy that empties the memory-side cache',
                   'valid_elements': n},
        'step': {'ms_min': float(np.min(cold_s)) * 1e3, 'gbps_28B': BYTES_UPDATE * n / t_cold / 1e9,
                 'frac_28B': BYTES_UPDATE * n / t_cold / 1e9 / HBM_PEAK_GBPS},
        'launch_sync_floor_us': floor_us,
        'host_us_in_step': host_us,
        'step_accounting_us': {
            'what': 'step = update launch + what any launch between two synchronisations costs (launch_sync_floor_us, '
                    'which already holds the host call of a launch) + what the host does in step() beyond such a call',
            'step': t_cold * 1e6, 'update_launch': t_upd_cold * 1e6, 'launch_sync_floor': floor_us,
            'host_call_of_step': host_us,
            'unaccounted': t_cold * 1e6 - t_upd_cold * 1e6 - floor_us,
            'steady_path_taken': opt._steady is not None,
        },
        'step_state_in_cache': {'what': 'the same step when nothing ran between two steps: the 256 MiB of state are '
                                        'still in the memory-side cache',
                                'ms_per_step': t_warm * 1e3, 'ms_min': float(np.min(warm_s)) * 1e3,
                                'frac_28B': BYTES_UPDATE * n / t_warm / 1e9 / HBM_PEAK_GBPS,
                                'update_launch_ms': t_upd_warm * 1e3,
                                'update_launch_frac': BYTES_UPDATE * n / t_upd_warm / 1e9 / HBM_PEAK_GBPS},
        'steps_back_to_back': {'what': f'{args.steps} steps between one pair of synchronisations, nothing between them',
                               'ms_per_step': t_queued * 1e3, 'frac_28B': BYTES_UPDATE * n / t_queued / 1e9 / HBM_PEAK_GBPS},
        'step_cold_cache': {'what': 'the line\'s own figure (kept under this name for comparison with earlier lines)',
                            'ms_per_step': t_cold * 1e3, 'ms_min': float(np.min(cold_s)) * 1e3,
                            'frac_28B': BYTES_UPDATE * n / t_cold / 1e9 / HBM_PEAK_GBPS},
        'roofline': {'kernel': 'adam_step_kernel', 'bound': 'hbm', 'achieved': BYTES_UPDATE * n / t_upd_cold / 1e9,
                     'peak': HBM_PEAK_GBPS, 'unit': 'GB/s', 'frac': BYTES_UPDATE * n / t_upd_cold / 1e9 / HBM_PEAK_GBPS,
                     'traffic': None, 'bytes_per_launch': BYTES_UPDATE * n, 'ms_per_launch': t_upd_cold * 1e3,
                     'timed_in': f'{extra - 1} extra steps after the timed ones, each behind the cache-emptying copy'},
    }
    if with_cpu:
        # the reference's own path for this configuration: torch.optim.Adam on CPU tensors, full size
        cp = torch.nn.Parameter(p.detach().cpu())
        copt = torch.optim.Adam([cp], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
        cp.grad = g.cpu()
        ts = []
        for _ in range(6):
            t0 = time.perf_counter()
            copt.step()
            ts.append(time.perf_counter() - t0)
        t = float(np.median(ts[1:]))
        out['cpu_baseline'] = {'value': n / t, 'unit': 'elements/s', 'cores': torch.get_num_threads(), 'kind': 'port',
                               'sample': 'the whole configuration: torch.optim.Adam on CPU fp32 tensors, median of 5 '
                                         'steps after 1 warm-up', 'extrapolation': 'none: full size',
                               'ms_per_step_sample': t * 1e3}
    return out


def velocity_line(args):
    """The reference's own optimizer micro-benchmark, profile/profile_optimizer.py:34-60, on one GPU:
    a flat fp32 parameter of 10**9 elements (zeros), a fresh fp32 gradient of ones before every
    step, HybridAdam(lr=1e-5), each ``optimizer.step()`` timed by the wall clock between two device
    synchronisations; velocity = steps * 1 (10**9 elements) / summed time.  elixir/search/
    simulator.py:128-129 hard-codes 50 (x10**9 elements/s per GPU, hardware not stated) as the result
    the reference's planner assumes.  28 B per element: read p, g, m, v, write p, m, v."""
    import elixir_amd as ea
    n = 10**9
    weight = torch.nn.Parameter(torch.zeros(n, device='cuda'))
    opt = ea.HybridAdam([weight], lr=1e-5)
    opt.kernel_events = {}
    step_s, adam_ms = [], []
    for i in range(args.warmup + args.steps):
        opt.zero_grad()
        weight.grad = torch.ones(n, dtype=torch.float, device='cuda')
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i >= args.warmup:
            step_s.append(dt)
            ev = opt.kernel_events['adam_step']
            adam_ms.append(ev[0].elapsed_time(ev[1]))
    opt.kernel_events = None
    # closed form after k steps from p = 0 with g = 1: m_hat = v_hat = 1, so every step moves p by -lr / (1 + eps)
    k = args.warmup + args.steps
    expect = -k * 1e-5 / (1.0 + 1e-8)
    got = weight.detach()[::max(1, n // 4096)].double().cpu().numpy()
    assert np.allclose(got, expect, rtol=1e-5, atol=0), (float(got[0]), expect)
    velocity = len(step_s) * (n / 1e9) / float(np.sum(step_s))
    t_step, t_upd = float(np.mean(step_s)), float(np.mean(adam_ms)) * 1e-3
    published = 50.0
    return {
        'metric': 'adam_velocity', 'value': velocity, 'unit': '1e9 elements/s', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': t_step * 1e3, 'higher_is_better': True, 'scaling': 'weak',
        'vs_baseline': velocity / published, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'velocity: flat fp32 parameter of 1e9 elements, fp32 gradient of ones, HybridAdam lr 1e-5 '
                               '(the reference\'s profile/profile_optimizer.py)', 'valid_elements': n,
                   'published_velocity': published, 'published_hardware': 'not stated by the reference'},
        'step': {'ms_min': float(np.min(step_s)) * 1e3, 'gbps_28B': BYTES_UPDATE * n / t_step / 1e9,
                 'frac_28B': BYTES_UPDATE * n / t_step / 1e9 / HBM_PEAK_GBPS},
        'roofline': {'kernel': 'adam_step_kernel', 'bound': 'hbm', 'achieved': BYTES_UPDATE * n / t_upd / 1e9,
                     'peak': HBM_PEAK_GBPS, 'unit': 'GB/s', 'frac': BYTES_UPDATE * n / t_upd / 1e9 / HBM_PEAK_GBPS,
                     'traffic': None, 'bytes_per_launch': BYTES_UPDATE * n, 'ms_per_launch': t_upd * 1e3},
    }


def chunk_set_line(args, workload: str, device, events_in_timed_steps: bool):
    """One chunk-set workload (c2, c4, c5) measured end to end; returns the JSON object of its line.

    ``events_in_timed_steps``: bracket the update launch with HIP events in every timed step (three
    records on the launch stream, about 6 us each: nothing next to 30 ms, 2 % of the GPT-2 step).
    Otherwise the timed steps run clean and every launch is timed in extra steps afterwards."""
    from elixir_amd import workloads
    t_build = time.perf_counter()
    built = workloads.build(workload, device)
    t_build = time.perf_counter() - t_build
    opt = built.optimizer
    opt.optim.blocks_per_cu = args.blocks_per_cu
    opt.blocks_per_cu = args.blocks_per_cu
    opt.graph_step = bool(args.graph)
    n_valid = built.n_valid

    step_s, upd_ms, stats_ms, adam_ms, refresh_ms = [], [], [], [], []
    if events_in_timed_steps:
        opt.optim.kernel_events = {}
    extra = 4
    for i in range(args.warmup + args.steps + extra):
        instrumented = i >= args.warmup + args.steps
        if instrumented and opt.kernel_events is None:
            opt.kernel_events = {}
            if opt.optim.kernel_events is None:
                opt.optim.kernel_events = {}
        built.land_gradients()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert opt.last_step_info['found_inf'] is False
        iev = opt.optim.kernel_events
        if instrumented:
            ev = opt.kernel_events
            upd_ms.append(ev['update'][0].elapsed_time(ev['update'][1]))
            stats_ms.append(ev['stats'][0].elapsed_time(ev['stats'][1]))
            if not events_in_timed_steps:
                adam_ms.append(iev['adam_step'][0].elapsed_time(iev['adam_step'][1]))
                refresh_ms.append(iev['refresh'][0].elapsed_time(iev['refresh'][1]) if 'refresh' in iev else 0.0)
        elif i >= args.warmup:
            step_s.append(dt)
            if events_in_timed_steps:
                adam_ms.append(iev['adam_step'][0].elapsed_time(iev['adam_step'][1]))
                refresh_ms.append(iev['refresh'][0].elapsed_time(iev['refresh'][1]) if 'refresh' in iev else 0.0)
    opt.kernel_events = None
    opt.optim.kernel_events = None
    upd_ms, stats_ms = upd_ms[1:], stats_ms[1:]    # the first instrumented step creates the event pairs
    if not events_in_timed_steps:
        adam_ms, refresh_ms = adam_ms[1:], refresh_ms[1:]

    t_step = float(np.mean(step_s))
    t_pair = float(np.mean(upd_ms)) * 1e-3        # update launch + padding refresh launch + host time between
    t_upd = float(np.mean(adam_ms)) * 1e-3         # adam_step_kernel alone
    t_refresh = float(np.mean(refresh_ms)) * 1e-3
    t_stats = float(np.mean(stats_ms)) * 1e-3      # stats launch + fold-and-decide launch
    upd_gbps = BYTES_UPDATE * n_valid / t_upd / 1e9
    plan = next(iter(opt.optim._plans.values())).plan
    traffic, traffic_source = traffic_fields(built.spec.name)
    out = {
        'metric': 'adam_elements_per_sec',
        'value': n_valid / t_step,
        'unit': 'elements/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': t_step * 1e3,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic',
        'config': {
            'workload': built.spec.name + ': ' + built.spec.description,
            'valid_elements': n_valid,
            'allocated_elements': built.n_alloc,
            'chunks': len(built.module.param_chunks),
            'tensors': len(opt.param_to_range),
            'loss_scale': built.spec.loss_scale,
            'combined_scale': opt.last_step_info['combined_scale'],
            'blocks_per_cu': args.blocks_per_cu,
            'graph_replay': bool(args.graph),
            'update_rows': len(plan.rows),
            'padding_in_update_launch': plan.refresh_rows is None and built.n_alloc > n_valid,
        },
        'step': {
            'ms_min': float(np.min(step_s)) * 1e3,
            'ms_median': float(np.median(step_s)) * 1e3,
            'gbps_30B': (BYTES_UPDATE + BYTES_STATS) * n_valid / t_step / 1e9,
            'frac_30B': (BYTES_UPDATE + BYTES_STATS) * n_valid / t_step / 1e9 / HBM_PEAK_GBPS,
            'gbps_touch_once_28B': BYTES_UPDATE * n_valid / t_step / 1e9,
            'frac_touch_once_28B': BYTES_UPDATE * n_valid / t_step / 1e9 / HBM_PEAK_GBPS,
        },
        'roofline': {
            'kernel': 'adam_step_kernel',
            'bound': 'hbm',
            'achieved': upd_gbps,
            'peak': HBM_PEAK_GBPS,
            'unit': 'GB/s',
            'frac': upd_gbps / HBM_PEAK_GBPS,
            'traffic': traffic,
            'traffic_source': traffic_source,
            'bytes_per_launch': BYTES_UPDATE * n_valid,
            'ms_per_launch': t_upd * 1e3,
            'timed_in': 'every timed step' if events_in_timed_steps else f'{extra - 1} extra steps after the timed ones',
        },
        'refresh_kernel': {
            'what': 'low-precision refresh of the chunk padding left out of the update launch',
            'ms_per_launch': t_refresh * 1e3,
            'update_plus_refresh_ms': t_pair * 1e3,
            'achieved_28B_over_both': BYTES_UPDATE * n_valid / t_pair / 1e9,
        },
        'stats_kernel': {
            'kernel': 'grad_stats_kernel+finish_decide_kernel',
            'achieved': BYTES_STATS * n_valid / t_stats / 1e9,
            'unit': 'GB/s',
            'frac': BYTES_STATS * n_valid / t_stats / 1e9 / HBM_PEAK_GBPS,
            'ms_per_launch': t_stats * 1e3,
        },
        'build_s': t_build,
    }
    if args.landing_steps > 0:
        out['fused_landing'] = fused_landing_leg(built, args.landing_steps)
    return out, built


def skip_step_leg(built, steps=20):
    """Configuration 3's timed part: the step that finds an overflow (on the c2 layout: one +inf planted in
    the gradients of the last chunk) -- stats launch, decision, and the update launch turned into the
    low-precision refresh of every shard; master / exp_avg / exp_avg_sq untouched, loss scale backed off.
    Bytes: 2 B per valid element (the flags) + 6 B per allocated element (4 B of master read, 2 B written).
    Runs last on its chunk set: it leaves the loss scale at its floor."""
    opt = built.optimizer
    pc = built.module.param_chunks[-1]
    keep = built.grads[-1][pc.utilized_size // 2].clone()
    built.grads[-1][pc.utilized_size // 2] = float('inf')
    master0 = pc.paired_chunk.shard[:4096].clone()
    ts = []
    for i in range(steps + 3):
        built.land_gradients()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
        assert opt.last_step_info['found_inf'] is True
    built.grads[-1][pc.utilized_size // 2] = keep
    assert torch.equal(master0, pc.paired_chunk.shard[:4096])
    t = float(np.mean(ts[3:]))
    nbytes = BYTES_STATS * built.n_valid + 6 * built.n_alloc
    return {'what': 'c3: the step that finds an overflow on the c2 layout (flags, decision, refresh of every shard; '
                    'nothing updated); the parity of the whole scenario is tests/test_gpu_configs.py',
            'steps': steps, 'ms_per_step': t * 1e3, 'ms_min': float(np.min(ts[3:])) * 1e3, 'bytes_per_step': nbytes,
            'gbps': nbytes / t / 1e9, 'frac': nbytes / t / 1e9 / HBM_PEAK_GBPS, 'loss_scale_after': opt.loss_scale}


def summary_of(line):
    """What the `configs` object keeps of a workload's line."""
    keep = {'workload': line['config']['workload'], 'valid_elements': line['config']['valid_elements'],
            'metric': line['metric'], 'value': line['value'], 'unit': line['unit'], 'steps': line['steps'],
            'ms_per_step': line['ms_per_step'], 'ms_min': line['step']['ms_min'],
            'roofline_frac_update_launch': line['roofline']['frac'],
            'update_launch_ms': line['roofline']['ms_per_launch'], 'update_launch_timed_in': line['roofline'].get('timed_in'),
            'update_launch_bytes': line['roofline']['bytes_per_launch'], 'update_launch_traffic': line['roofline'].get('traffic'),
            'update_launch_traffic_source': line['roofline'].get('traffic_source')}
    for k in ('frac_30B', 'frac_touch_once_28B', 'frac_28B'):
        if k in line['step']:
            keep['step_' + k] = line['step'][k]
    if 'stats_kernel' in line:
        keep['stats_launch_ms'] = line['stats_kernel']['ms_per_launch']
        keep['stats_frac'] = line['stats_kernel']['frac']
    if 'fused_landing' in line:
        keep['step_after_fused_landing_ms'] = line['fused_landing']['ms_per_step']
        keep['step_after_fused_landing_frac_28B'] = line['fused_landing']['step_frac_28B']
        keep['step_after_per_chunk_landing_ms'] = line['fused_landing']['per_chunk_landing']['ms_per_step']
        keep['per_chunk_landing'] = line['fused_landing']['per_chunk_landing']
        keep['payload_landing_ms'] = line['fused_landing']['land_kernel']['ms_per_launch']
        keep['payload_landing_frac'] = line['fused_landing']['land_kernel']['frac']
        keep['per_tensor_landing'] = line['fused_landing']['per_tensor_landing']
    if line.get('vs_baseline') is not None:
        keep['vs_baseline'] = line['vs_baseline']
    if 'step_cold_cache' in line:
        keep['step_cold_cache_ms'] = line['step_cold_cache']['ms_per_step']
        keep['step_state_in_cache_ms'] = line['step_state_in_cache']['ms_per_step']
        keep['steps_back_to_back_ms'] = line['steps_back_to_back']['ms_per_step']
        keep['launch_sync_floor_us'] = line['launch_sync_floor_us']
        keep['host_us_in_step'] = line['host_us_in_step']
        keep['step_accounting_us'] = line['step_accounting_us']
    if 'cpu_baseline' in line:
        keep['cpu_baseline'] = line['cpu_baseline']
    return keep


def free_device_memory():
    import gc
    gc.collect()
    torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--workload', default='c5', choices=['c1', 'c2', 'c4', 'c5', 'velocity'])
    ap.add_argument('--cpu-sample', type=int, default=256 << 20, help='elements of the CPU baseline sample; 0 skips it')
    ap.add_argument('--blocks-per-cu', type=int, default=0,
                    help='cap on resident update workgroups per compute unit (0 = library default)')
    ap.add_argument('--graph', action='store_true',
                    help='replay the launches of a step from a recorded HIP graph (ElixirOptimizer.graph_step)')
    ap.add_argument('--no-configs', action='store_true',
                    help='only the headline workload: leave the `configs` object with the other configurations out')
    ap.add_argument('--calibrate-copy', type=float, default=0.0,
                    help='instead of the benchmark, run three plain device copies of this many GiB (a kernel of '
                    'known traffic, to scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run) and exit')
    ap.add_argument('--landing-steps', type=int, default=5,
                    help='steps of the additional leg in which the gradients arrive through the fused landing '
                    'launch (0: skip the leg)')
    ap.add_argument('--offload-step', type=int, default=0, metavar='MI',
                    help='only time the step over one host-resident chunk pair of MI Mi elements and exit')
    ap.add_argument('--offload-gather', type=int, default=0, metavar='MI',
                    help='only time the gather source copy of one host-resident chunk of MI Mi elements and exit')
    args = ap.parse_args()

    if args.gpus != 1:
        print('bench.py measures the optimizer step on ONE GPU (each rank owns whole shards; there is no '
              'multi-GPU path in this build): run with --gpus 1', file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print('bench.py needs a GPU: the optimizer step has no CPU path', file=sys.stderr)
        sys.exit(2)

    from elixir_amd.build import ensure_built
    ensure_built()    # loads what is built; compiles only a tree that was never built

    if args.offload_step > 0:
        print(json.dumps(offload_step_leg(args.offload_step)))
        return
    if args.offload_gather > 0:
        print(json.dumps(offload_gather_leg(args.offload_gather)))
        return

    if args.calibrate_copy > 0:
        n = int(args.calibrate_copy * (1 << 30)) // 4
        src = torch.rand(n, device='cuda')
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({'calibrate_copy_bytes_read': n * 4, 'calibrate_copy_bytes_written': n * 4, 'copies': 3}))
        return

    from elixir_amd import _abi
    _abi.load()
    device = torch.device('cuda', 0)
    torch.cuda.set_device(device)
    if args.workload == 'c1':
        print(json.dumps(config1_line(args, with_cpu=args.cpu_sample > 0)))
        return
    if args.workload == 'velocity':
        print(json.dumps(velocity_line(args)))
        return

    out, built = chunk_set_line(args, args.workload, device, events_in_timed_steps=args.workload == 'c5')
    if args.cpu_sample > 0:
        out['cpu_baseline'] = cpu_baseline(built, args.cpu_sample)
    if args.workload == 'c2':
        out['skip_step'] = skip_step_leg(built, steps=max(3, args.steps))
    del built
    free_device_memory()

    if args.workload == 'c5' and not args.no_configs:
        # the other configurations in the same run (fewer steps each: a few hundred milliseconds of GPU time)
        configs = {}
        small = argparse.Namespace(**vars(args))
        small.landing_steps = min(args.landing_steps, 5)
        for name, steps in (('c4', 20), ('c2', 50)):
            small.steps, small.warmup = steps, 5
            line, b = chunk_set_line(small, name, device, events_in_timed_steps=False)
            if name == 'c2':
                configs['c3'] = skip_step_leg(b)
                if args.cpu_sample > 0:
                    line['cpu_baseline'] = cpu_baseline_whole_set(b)
            del b
            free_device_memory()
            configs[name] = summary_of(line)
        small.steps, small.warmup = 50, 5
        configs['c1'] = summary_of(config1_line(small, with_cpu=args.cpu_sample > 0))
        free_device_memory()
        small.steps, small.warmup = 10, 2
        configs['velocity'] = summary_of(velocity_line(small))
        free_device_memory()
        out['configs'] = configs
    print(json.dumps(out))


if __name__ == '__main__':
    main()
