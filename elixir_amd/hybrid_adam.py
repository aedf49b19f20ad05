"""``HybridAdam``: the Adam / AdamW optimizer the reference hands to its wrapper
(``elixir/wrapper/optimizer.py:19,216``), with the same constructor and the same
``step(closure=None, div_scale=-1)`` call, running on the HIP kernels of ``libelx_hip.so``.

Two ways in:

* standalone, on ordinary fp32 CUDA parameters with ``.grad`` set (fp32, fp16 or bf16 gradients) --
  the flat-parameter use of ``profile/profile_optimizer.py:34-60``;
* bound to chunk storage by ``ElixirOptimizer`` (``bind_chunks``): master weights, exp_avg and
  exp_avg_sq are flat fp32 buffers per chunk, gradients are read from the low-precision shards and
  the refreshed low-precision parameters are written back by the same launch.

Either way one step is one launch over every tensor of every parameter group.  The arithmetic
follows ``torch.optim.Adam`` / ``AdamW`` (float64 host scalars narrowed to fp32, same op order);
there is no CPU path.  "Hybrid" in the reference means GPU kernels for device-resident shards and
a CPU Adam for host-resident ones; here shards in pinned host memory go into the same launch and
are read and written in place over the host link, shards in pageable host memory are refused.
"""
import math
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
from torch.optim import optimizer as _torch_optimizer

from . import _abi
from .chunk import gpu_device, Chunk, DeviceTable, dtype_code
from .launch_plan import FlatBuffer, LaunchPlan, build_plan


def make_hyper_record(lr: float, beta1: float, beta2: float, eps: float, weight_decay: float, step: int,
                      bias_correction: bool, adamw_mode: bool) -> np.ndarray:
    """Host scalars of one (group, step) pair -- torch/optim/adam.py:414-430,528-535 -- narrowed
    to fp32 where a tensor op would narrow a Python scalar."""
    rec = np.zeros(1, dtype=_abi.HYPER_DTYPE)
    bc1 = 1.0 - beta1**step if bias_correction else 1.0
    bc2 = 1.0 - beta2**step if bias_correction else 1.0
    flags = 0
    decay_mul, l2_wd = 1.0, 0.0
    if weight_decay != 0:
        if adamw_mode:
            decay_mul = 1.0 - lr * weight_decay
        else:
            l2_wd = weight_decay
            flags |= _abi.ELX_HYPER_L2
    w1 = np.float32(1.0 - beta1)
    if w1 < np.float32(0.5):
        lerp_w = w1
    else:
        lerp_w = np.float32(w1 - np.float32(1.0))
        flags |= _abi.ELX_HYPER_LERP_FROM_G
    rec['decay_mul'] = decay_mul
    rec['l2_wd'] = l2_wd
    rec['lerp_w'] = lerp_w
    rec['beta2'] = beta2
    rec['omb2'] = 1.0 - beta2
    rec['bc2_sqrt'] = math.sqrt(bc2)
    rec['eps'] = eps
    rec['neg_step'] = -(lr / bc1)
    rec['flags'] = flags
    return rec


_HYPER_RECORDS: Dict = {}


def hyper_record_cached(key: Tuple, adamw_mode: bool) -> np.ndarray:
    """``make_hyper_record`` for ``key = (lr, beta1, beta2, eps, weight_decay, step, bias_correction)``, kept:
    a step looks up the records the step before it has already computed while its launch was running."""
    rec = _HYPER_RECORDS.get((key, adamw_mode))
    if rec is None:
        if len(_HYPER_RECORDS) > 4096:
            _HYPER_RECORDS.clear()
            _HYPER_ADDRESSES.clear()
        lr, b1, b2, eps, wd, step, bc = key
        rec = _HYPER_RECORDS[(key, adamw_mode)] = make_hyper_record(lr, b1, b2, eps, wd, step, bc, adamw_mode)
        rec.flags.writeable = False    # shared between steps: nobody edits it
    return rec


_HYPER_ADDRESSES: Dict = {}


def hyper_record_address(key: Tuple, adamw_mode: bool) -> int:
    """Host address of the cached record for ``key`` (the record stays alive in the cache, which is emptied
    together with this table)."""
    ptr = _HYPER_ADDRESSES.get((key, adamw_mode))
    if ptr is None:
        rec = hyper_record_cached(key, adamw_mode)    # may empty both tables first
        ptr = _HYPER_ADDRESSES[(key, adamw_mode)] = rec.ctypes.data
    return ptr


def _raw_current_stream(device: torch.device) -> int:
    """The current stream's handle.  torch keeps a direct getter for it, a third of the cost of building a
    ``torch.cuda.Stream`` object first; without that getter the object's handle is taken."""
    getter = getattr(torch._C, '_cuda_getCurrentRawStream', None)
    if getter is not None:
        return getter(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _SteadyStep:
    """A standalone step over the same buffers as the step before it, all of them one step further: the
    walk over the parameters, the launch plan and the tables are those of the last step, and all that is
    new are the hyper records (computed while the last launch was running).  What it keeps lets the next
    ``step()`` go from its first line to the launch in a few microseconds -- on a 16 Mi-element parameter
    the launch itself takes under 70, and whatever the host needs in front of it the device spends idle."""

    __slots__ = ('watch', 'layout', 'states', 'step', 'group_of_hyper', 'dplan', 'grad_code', 'device', 'call', 'fixed',
                 'tail', 'flags', 'pack', 'pack_ptr')

    def __init__(self, watch, layout, prep: '_Prepared', step: int, group_of_hyper):
        plan = prep.dplan.plan
        self.watch, self.layout, self.states, self.step = watch, layout, prep.states, step
        self.group_of_hyper = group_of_hyper      # group index of every hyper record, in table order
        self.dplan, self.grad_code, self.device = prep.dplan, prep.grad_code, prep.device
        self.call = _abi.load().elx_adam_step_put_mt
        self.fixed = (prep.dplan.rows.ptr, len(plan.rows), prep.dplan.segs.ptr, len(plan.segs))
        self.tail = (plan.info.total_tiles, plan.info.max_tiles)
        self.flags = plan.info.flags
        n = len(group_of_hyper)
        self.pack = np.zeros(n, dtype=_abi.HYPER_DTYPE) if n > 1 else None    # several records: gathered here
        self.pack_ptr = self.pack.ctypes.data if n > 1 else 0


_NO_HOOKS: Dict = {}


def _global_step_hooks():
    """torch's process-wide optimizer step hooks (``register_optimizer_step_pre_hook`` /
    ``..._post_hook``).  They live in private module attributes of torch.optim.optimizer; a torch that
    names them differently has no such hooks as far as this class can tell."""
    return (getattr(_torch_optimizer, '_global_optimizer_pre_hooks', _NO_HOOKS),
            getattr(_torch_optimizer, '_global_optimizer_post_hooks', _NO_HOOKS))


class _CachedTable:
    """Device copy of a host table, re-uploaded only when the host contents change."""

    def __init__(self):
        self.table: Optional[DeviceTable] = None

    def get(self, host: np.ndarray, device: torch.device) -> DeviceTable:
        t = self.table
        if t is None or t.dev.device != device or t.host.shape != host.shape or t.host.tobytes() != host.tobytes():
            self.table = DeviceTable(host.copy(), device)
        return self.table


class _HyperTable:
    """The device table of the hyper records of a step.  The records change every step (bias
    corrections); they reach the device in the arguments of a one-wavefront launch on the launch stream
    (``elx_put_hypers``): nothing to stage, nothing to wait for, and the host array is free at once."""

    def __init__(self):
        self.dev: Optional[torch.Tensor] = None

    def reserve(self, nbytes: int, device: torch.device) -> int:
        if self.dev is None or self.dev.device != device or self.dev.numel() < nbytes:
            self.dev = torch.empty(max(4096, nbytes), dtype=torch.uint8, device=device)
        return self.dev.data_ptr()

    def put(self, host: np.ndarray, device: torch.device) -> int:
        ptr = self.reserve(host.nbytes, device)
        _abi.put_hypers(host, ptr, torch.cuda.current_stream(device).cuda_stream)
        return ptr


class _DevicePlan:
    """A launch plan and its tables in device memory."""

    def __init__(self, plan: LaunchPlan, device: torch.device):
        self.plan = plan
        self.rows = DeviceTable(plan.rows, device) if len(plan.rows) else None
        self._gated_rows: Optional[DeviceTable] = None
        self.armed: Optional[torch.Tensor] = None    # one device word: whether the gated copy holds zeros right now
        self.segs = DeviceTable(plan.segs, device) if len(plan.segs) else None
        self.refresh = DeviceTable(plan.refresh_rows, device) if plan.refresh_rows is not None else None
        self.refresh_aligned = True
        if plan.refresh_rows is not None:
            self.refresh_aligned = bool(
                np.all(plan.refresh_rows['lowp_out'] % 16 == 0) and np.all(plan.refresh_rows['master'] % 16 == 0))


    @property
    def gated_rows(self) -> Optional[DeviceTable]:
        """A second device copy of the update rows, made when a step is first decided on the device: the table
        of the gated update launch, whose n_valid column the decision launch rewrites at every step (zeros on a
        skip).  ``rows`` itself is never written: host-decided launches read it."""
        if self._gated_rows is None and self.rows is not None:
            self._gated_rows = DeviceTable(self.plan.rows, self.rows.dev.device)
            self.armed = torch.zeros(1, dtype=torch.int32, device=self.rows.dev.device)
        return self._gated_rows


class ChunkBinding:
    """Where the fake parameters of ``ElixirOptimizer`` live: for each optimizer chunk the paired
    low-precision chunk, the flat m / v buffers and the slices the optimizer owns."""

    def __init__(self, ranges: Dict[torch.nn.Parameter, Tuple[Chunk, int, int]]):
        # optimizer chunk -> index in the launch
        self.chunks: List[Chunk] = sorted({c for c, _, _ in ranges.values()})
        self.chunk_index = {c: i for i, c in enumerate(self.chunks)}
        self.ranges = ranges
        self.flat_m: Dict[Chunk, torch.Tensor] = {}
        self.flat_v: Dict[Chunk, torch.Tensor] = {}
        self.zero_grads = False        # the allocation step: gradients are zero, nothing is written back
        self.fused_writeback = False   # set by step(): the launch refreshed the low-precision shards
        for c in self.chunks:
            assert c.paired_chunk is not None, 'chunks should be paired before training'
            assert c.chunk_dtype == torch.float32
            assert c.paired_chunk.shard_device == c.shard_device

    def require_gpu(self) -> None:
        """Every buffer of the launch must be reachable by the kernels: device memory, or pinned
        host memory (which they read and write in place over the host link)."""
        if not torch.cuda.is_available():
            raise RuntimeError('HybridAdam runs on the GPU: no device is available')
        for c in self.chunks:
            for shard in (c.shard, c.paired_chunk.shard):
                if not (shard.is_cuda or shard.is_pinned()):
                    raise RuntimeError('HybridAdam runs on the GPU: shards must live in device memory or in '
                                       'pinned host memory (cpu_pin_memory=True); pageable host memory cannot be '
                                       'reached by the kernels')

    def launch_device(self) -> torch.device:
        for c in self.chunks:
            if c.shard.is_cuda:
                return c.shard_device
        return gpu_device()

    def moments(self, chunk: Chunk) -> Tuple[torch.Tensor, torch.Tensor]:
        """The flat exp_avg / exp_avg_sq of an optimizer chunk, allocated beside its shard: in device
        memory, or in pinned host memory for a host-resident shard."""
        if chunk not in self.flat_m:
            if chunk.shard.is_cuda or not torch.cuda.is_available():
                kw = dict(device=chunk.shard_device)
            else:
                kw = dict(pin_memory=True)
            self.flat_m[chunk] = torch.zeros(chunk.shard_size, dtype=torch.float32, **kw)
            self.flat_v[chunk] = torch.zeros(chunk.shard_size, dtype=torch.float32, **kw)
        return self.flat_m[chunk], self.flat_v[chunk]


class _Prepared:
    """Everything a step needs that does not depend on the gradient flags: built while the stats
    launch is still running, consumed (and only then committed to the optimizer state) by step()."""

    def __init__(self, dplan, hyper_host, grad_code, lowp_code, device, states, hyper_keys=(), hyper_index=()):
        self.dplan: _DevicePlan = dplan
        self.hyper_index = hyper_index        # per entry of ``states``: which hyper record it is updated with
        self.hyper_host: np.ndarray = hyper_host
        self.hyper_keys = tuple(hyper_keys)    # (lr, beta1, beta2, eps, weight_decay, step, bias_correction) per record
        self.grad_code, self.lowp_code, self.device = grad_code, lowp_code, device
        self.states: List[Dict] = states      # per-parameter state dicts whose 'step' advances on commit
        self.d_hypers: int = 0
        self.sig = None


class HybridAdam(torch.optim.Optimizer):
    """Adam / AdamW with a fused gradient unscale.

    Arguments follow ColossalAI's ``HybridAdam``:
        model_params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, weight_decay=0,
        adamw_mode=True (decoupled decay; False adds ``wd * p`` to the gradient),
        nvme_offload_fraction / nvme_offload_dir (accepted; offloading is not supported here).

    ``step(closure=None, div_scale=-1)``: gradients are divided by ``div_scale`` when it is
    positive -- the combined loss scale and clipping coefficient of optimizer.py:166-183.
    """

    def __init__(self,
                 model_params,
                 lr: float = 1e-3,
                 bias_correction: bool = True,
                 betas: Tuple[float, float] = (0.9, 0.999),
                 eps: float = 1e-8,
                 weight_decay: float = 0,
                 adamw_mode: bool = True,
                 nvme_offload_fraction: float = 0.0,
                 nvme_offload_dir: Optional[str] = None,
                 **defaults):
        if nvme_offload_fraction != 0.0:
            raise NotImplementedError('NVMe offload of optimizer states is not supported')
        default_args = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, bias_correction=bias_correction)
        super().__init__(model_params, default_args)
        self.adamw_mode = adamw_mode
        self.blocks_per_cu = 0    # cap on resident update workgroups per compute unit; 0: library default
        self._binding: Optional[ChunkBinding] = None
        self._plans: Dict = {}                      # plan key -> _DevicePlan
        self._hyper_table_dev = _HyperTable()
        self._prepared: Optional[_Prepared] = None
        self._launched: Optional[_Prepared] = None   # launched with defer_commit, not yet committed or aborted
        self._bound_entries = None                  # cached walk over the bound fake parameters
        self._standalone_cache = None               # cached walk over standalone parameters and their gradients
        self._steady: Optional[_SteadyStep] = None   # a standalone step that can repeat the one before it
        # when set to a dict, step() records (begin, end) torch.cuda.Event pairs under 'adam_step' and 'refresh'
        self.kernel_events = None

    # ------------------------------------------------------------------ chunk binding

    def bind_chunks(self, ranges: Dict[torch.nn.Parameter, Tuple[Chunk, int, int]]) -> ChunkBinding:
        """Called by ``ElixirOptimizer``: ``ranges[fake_param] = (optim_chunk, begin, end)``."""
        self._binding = ChunkBinding(ranges)
        self._bound_entries = None
        self._plans.clear()
        return self._binding

    @property
    def binding(self) -> Optional[ChunkBinding]:
        return self._binding

    # ------------------------------------------------------------------ the step

    @staticmethod
    def _group_key(group: Dict, step: int):
        beta1, beta2 = group['betas']
        return (group['lr'], beta1, beta2, group['eps'], group['weight_decay'], step, group['bias_correction'])

    def _hyper_index(self, hypers: Dict, group: Dict, step: int) -> int:
        key = self._group_key(group, step)
        idx = hypers.get(key)
        if idx is None:
            idx = len(hypers)
            hypers[key] = idx
        return idx

    def _device_plan(self, key, buffers_fn, grad_dtype, grad_code, lowp_code, n_hypers, device,
                     device_resident: bool = True) -> _DevicePlan:
        dplan = self._plans.get(key)
        if dplan is None:
            if len(self._plans) > 8:
                self._plans.clear()
            esize = 4 if grad_dtype == torch.float32 else 2
            dplan = _DevicePlan(build_plan(buffers_fn(), esize, esize, n_hypers, grad_code, lowp_code,
                                           device_resident=device_resident), device)
            self._plans[key] = dplan
        return dplan

    def prepare_step(self, upload: bool = True) -> None:
        """Builds the tables of the next step without touching the optimizer state, so that a caller
        can overlap this host work with device work whose result decides whether the step happens
        (``ElixirOptimizer`` calls it between launching and reading the gradient flags).  The next
        ``step()`` consumes what was prepared; ``discard_prepared()`` drops it.  ``upload`` False leaves
        the hyper records on the host: the caller gets them to the device its own way (or the launch
        uploads them after all)."""
        sig = self._prepare_signature()
        if self._prepared is not None and sig is not None and self._prepared.sig == sig:
            prep = self._prepared    # prepared ahead of time (ElixirOptimizer.backward does) and still valid
        else:
            hypers: Dict = {}
            if self._binding is not None:
                self._prepared = self._prepare_bound(hypers)
            else:
                self._prepared = self._prepare_standalone(hypers)
            prep = self._prepared
            if prep is not None:
                prep.sig = sig
        if prep is not None and upload and not prep.d_hypers:
            prep.d_hypers = self._hyper_table_dev.put(prep.hyper_host, prep.device)

    def adopt_prepared(self) -> None:
        """The prepared step counts as launched without a launch from here: its launches were recorded
        earlier (a HIP graph of the same tables) and the caller replays them."""
        self._launched, self._prepared = self._prepared, None

    def _prepare_signature(self):
        """Everything a prepared step of bound chunks depends on besides the step counts (which only
        change when a prepared step is consumed or a state is loaded, and both drop it): the group
        hyper-parameters, the group sizes and the kind of step.  None for standalone parameters,
        whose gradient buffers change from step to step."""
        if self._binding is None:
            return None
        return (self._binding.zero_grads,
                tuple((len(g['params']), ) + self._group_key(g, 0) for g in self.param_groups))

    def discard_prepared(self) -> None:
        self._prepared = None

    def _hyper_table(self, hypers: Dict) -> np.ndarray:
        records = [hyper_record_cached(key, self.adamw_mode) for key in hypers.keys()]
        return records[0] if len(records) == 1 else np.concatenate(records)

    def step(self, closure=None, div_scale: float = -1, *, gated: bool = False, defer_commit: bool = False,
             armed_rows: bool = False):
        """``gated``: the unscale parameters and the skip flag are read on the device from the gate
        words of the prepared hyper table, where ``elx_finish_decide`` has put them (``div_scale`` is then
        ignored).  ``armed_rows`` (with ``gated``): the launch reads the second copy of the update rows, whose
        counts of valid elements the decision launch has just rewritten (``_DevicePlan.gated_rows``).  ``defer_commit``: launch only; the caller finishes with ``commit_step()`` once it
        knows that the step happened, or ``abort_step()`` when the device decided to skip.

        torch wraps every optimizer's ``step`` in a profiler scope and its hook dispatch, tens of
        microseconds during which the device waits; this class opts out of that wrapper (the ``hooked``
        mark below) and runs registered step hooks itself, in torch's order."""
        global_pre, global_post = _global_step_hooks()
        if not (global_pre or global_post or self._optimizer_step_pre_hooks or self._optimizer_step_post_hooks):
            return self.launch_step(closure, div_scale, gated=gated, defer_commit=defer_commit, armed_rows=armed_rows)
        pre = list(global_pre.values()) + list(self._optimizer_step_pre_hooks.values())
        post = list(self._optimizer_step_post_hooks.values()) + list(global_post.values())
        args, kwargs = (closure, div_scale), dict(gated=gated, defer_commit=defer_commit)
        if armed_rows:
            kwargs['armed_rows'] = True
        for hook in pre:
            result = hook(self, args, kwargs)
            if result is not None:
                if not (isinstance(result, tuple) and len(result) == 2):
                    raise RuntimeError(f'{hook} must return None or a tuple of (new_args, new_kwargs), but got {result}.')
                args, kwargs = result
        out = self.launch_step(*args, **kwargs)
        for hook in post:
            hook(self, args, kwargs)
        return out

    step.hooked = True    # torch.optim.Optimizer leaves a step marked like this unwrapped

    def launch_step(self, closure=None, div_scale: float = -1, *, gated: bool = False, defer_commit: bool = False,
                    armed_rows: bool = False):
        """The launches of one step (``step`` without the hook dispatch).  Nothing here builds an autograd
        graph, so no ``no_grad`` scope is entered either."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        steady = self._steady
        if steady is not None:
            if (self._prepared is None and not gated and not defer_commit and self.kernel_events is None
                    and self._steady_still_holds(steady)):
                self._launch_steady(steady, div_scale)
                return loss
            self._steady = None
        if self._prepared is None:
            self.prepare_step(upload=False)    # the records go out with the launch below
        prep, self._prepared = self._prepared, None
        if prep is None:
            return loss

        plan = prep.dplan.plan
        stream = torch.cuda.current_stream(prep.device).cuda_stream
        events = self.kernel_events
        together = False    # hyper records and update in one call: the two launches go out back to back
        if not prep.d_hypers:
            if gated or events is not None or prep.dplan.rows is None:
                prep.d_hypers = self._hyper_table_dev.put(prep.hyper_host, prep.device)
            else:
                prep.d_hypers = self._hyper_table_dev.reserve(prep.hyper_host.nbytes, prep.device)
                together = True
        if prep.dplan.rows is not None:
            if events is not None:
                if 'adam_step' not in events:    # created once, recorded again every step
                    events['adam_step'] = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                events['adam_step'][0].record()
            if gated:
                rows = prep.dplan.gated_rows if armed_rows else prep.dplan.rows
                _abi.adam_step_gated_mt(rows.ptr, len(plan.rows), prep.dplan.segs.ptr, len(plan.segs),
                                        prep.d_hypers, len(prep.hyper_host), plan.info, prep.grad_code,
                                        prep.lowp_code, self.blocks_per_cu, stream)
            elif together:
                _abi.adam_step_put_mt(prep.dplan.rows.ptr, len(plan.rows), prep.dplan.segs.ptr, len(plan.segs),
                                      prep.hyper_host, prep.d_hypers, plan.info, float(div_scale), prep.grad_code,
                                      prep.lowp_code, self.blocks_per_cu, stream)
            else:
                _abi.adam_step_mt(prep.dplan.rows.ptr, len(plan.rows), prep.dplan.segs.ptr, len(plan.segs),
                                  prep.d_hypers, len(prep.hyper_host), plan.info, float(div_scale), prep.grad_code,
                                  prep.lowp_code, self.blocks_per_cu, stream)
            if events is not None:
                events['adam_step'][1].record()
        if prep.dplan.refresh is not None:
            if events is not None and 'refresh' not in events:
                # the refresh is bracketed by the end of the update launch and its own end event
                begin = events['adam_step'][1] if 'adam_step' in events else torch.cuda.Event(enable_timing=True)
                events['refresh'] = (begin, torch.cuda.Event(enable_timing=True))
                if 'adam_step' not in events:
                    begin.record()
            _abi.writeback_mt(prep.dplan.refresh.ptr, len(plan.refresh_rows), prep.lowp_code, plan.refresh_max_elems,
                              prep.dplan.refresh_aligned, stream)
            if events is not None:
                events['refresh'][1].record()
        self._launched = prep
        if not defer_commit:
            self.commit_step()
            if together and self._binding is None and prep.dplan.refresh is None:
                self._remember_steady(prep)
        return loss

    # ---- a standalone step that repeats the one before it

    def _remember_steady(self, prep: '_Prepared') -> None:
        """After a standalone step whose records rode in its launch: keep what the next step can reuse if
        nothing but the step counts has changed by then."""
        cache = self._standalone_cache
        if cache is None or not prep.states or len(prep.hyper_keys) > _abi.MAX_ARG_HYPERS:
            return
        watch, layout, (items, _, _) = cache
        step = prep.states[0]['step']
        if any(st['step'] != step for st in prep.states):
            return    # per-parameter step counts differ: the records would have to be matched to parameters again
        group_of_hyper = [None] * len(prep.hyper_keys)
        for (state, gi, _), h in zip(items, prep.hyper_index):
            if group_of_hyper[h] is None:
                group_of_hyper[h] = gi
            elif group_of_hyper[h] != gi:
                return    # two groups share one record: a change in one of them would need a new plan
        self._steady = _SteadyStep(watch, layout, prep, step, group_of_hyper)

    def _steady_still_holds(self, steady: _SteadyStep) -> bool:
        groups = self.param_groups
        if len(groups) != len(steady.layout):
            return False
        for group, count in zip(groups, steady.layout):
            if len(group['params']) != count:
                return False
        if not self._watch_holds(steady.watch):
            return False
        step = steady.step
        for state in steady.states:
            if state['step'] != step:
                return False
        return True

    def _launch_steady(self, steady: _SteadyStep, div_scale: float) -> None:
        groups = self.param_groups
        step = steady.step + 1
        if steady.pack is None:
            key = self._group_key(groups[steady.group_of_hyper[0]], step)
            ptr = hyper_record_address(key, self.adamw_mode)
            keys = (key, )
        else:
            keys = tuple(self._group_key(groups[gi], step) for gi in steady.group_of_hyper)
            # (two groups whose hyper-parameters have become equal would share a record in a freshly built plan;
            # this plan keeps one record each, which is the same arithmetic)
            for h, key in enumerate(keys):
                steady.pack[h] = hyper_record_cached(key, self.adamw_mode)[0]
            ptr = steady.pack_ptr
        stream = _raw_current_stream(steady.device)
        d_hypers = self._hyper_table_dev.reserve(len(keys) * _abi.HYPER_DTYPE.itemsize, steady.device)
        code = steady.call(*steady.fixed, ptr, d_hypers, len(keys), *steady.tail, float(div_scale), steady.grad_code,
                           _abi.ELX_NONE, steady.flags, self.blocks_per_cu, stream)
        if code != 0:
            _abi.check('elx_adam_step_put_mt', code)
        # the launch is out: bookkeeping, and the records of the step after this one
        for state in steady.states:
            state['step'] = step
        steady.step = step
        for (lr, b1, b2, eps, wd, st, bc) in keys:
            hyper_record_address((lr, b1, b2, eps, wd, st + 1, bc), self.adamw_mode)

    def commit_step(self) -> None:
        """The launched step happened: step counts advance (after the launches, so that the device is
        not kept waiting for host bookkeeping)."""
        prep, self._launched = self._launched, None
        if prep is None:
            return
        for state in prep.states:
            state['step'] += 1
        if self._binding is not None and prep.lowp_code != _abi.ELX_NONE:
            self._binding.fused_writeback = True
        # the records of the next step, computed now, while the device is busy with this one
        for (lr, b1, b2, eps, wd, step, bc) in prep.hyper_keys:
            hyper_record_cached((lr, b1, b2, eps, wd, step + 1, bc), self.adamw_mode)

    def abort_step(self) -> None:
        """The launched step found the skip flag set on the device: nothing was updated and no step
        count advances; the launches refreshed every low-precision element they cover."""
        prep, self._launched = self._launched, None
        if prep is not None and self._binding is not None and prep.lowp_code != _abi.ELX_NONE:
            self._binding.fused_writeback = True

    # ---- bound to chunk storage

    # ---- checkpoint of the optimizer state

    def _ensure_state(self) -> None:
        """Bound fake parameters get their (step, exp_avg, exp_avg_sq) entries -- views of the flat
        per-chunk moments -- before the first step, so that a fresh optimizer can save or load."""
        if self._binding is not None:
            self._walk_bound()

    def state_dict(self):
        """torch's packed layout (``state`` keyed by the running index of the parameter over the
        groups, ``param_groups`` with those indices).  ``exp_avg`` / ``exp_avg_sq`` are CPU copies,
        detached from the flat storage; with bound chunks they are the 1-D slices this process owns."""
        self._ensure_state()
        packed = super().state_dict()
        # torch hands out the optimizer's own per-parameter dicts: build new ones, never edit those
        packed['state'] = {
            pid: {key: (value.detach().to('cpu', copy=True) if torch.is_tensor(value) else value)
                  for key, value in st.items()}
            for pid, st in packed['state'].items()
        }
        return packed

    def load_state_dict(self, state_dict) -> None:
        """Restores what ``state_dict`` saved, IN PLACE: the moments are copied into the flat
        per-chunk buffers (or the existing per-parameter tensors) the update launch reads, never
        replaced by new tensors; step counts and group hyper-parameters are taken over."""
        self._ensure_state()
        groups, saved_groups = self.param_groups, state_dict['param_groups']
        if len(groups) != len(saved_groups) or any(
                len(g['params']) != len(sg['params']) for g, sg in zip(groups, saved_groups)):
            raise ValueError('loaded state dict has a different number of parameter groups or parameters')
        id_to_param = {}
        for g, sg in zip(groups, saved_groups):
            for p, pid in zip(g['params'], sg['params']):
                id_to_param[pid] = p
            for key, value in sg.items():
                if key != 'params':
                    g[key] = value
        for pid, saved in state_dict['state'].items():
            p = id_to_param[int(pid)]
            state = self.state[p]
            for key in ('exp_avg', 'exp_avg_sq'):
                if key not in saved:
                    continue
                if key not in state:    # a standalone parameter that has not stepped yet
                    state[key] = torch.zeros_like(p, memory_format=torch.preserve_format)
                src = saved[key]
                if src.numel() != state[key].numel():
                    raise ValueError(f'parameter {pid}: saved {key} has {src.numel()} elements, '
                                     f'this optimizer holds {state[key].numel()}')
                state[key].copy_(src.reshape(state[key].shape))
            step = saved.get('step', 0)
            state['step'] = int(step.item()) if torch.is_tensor(step) else int(step)
        self._prepared = None
        self._standalone_cache = None
        self._steady = None

    def _walk_bound(self):
        """(state dict, group index, chunk index, begin, end) per bound fake parameter, in group order."""
        b = self._binding
        signature = tuple(len(g['params']) for g in self.param_groups)
        if self._bound_entries is not None and self._bound_entries[0] == signature:
            return self._bound_entries[1]
        entries = []
        for gi, group in enumerate(self.param_groups):
            for p in group['params']:
                if p not in b.ranges:
                    raise RuntimeError('a parameter of this optimizer is not part of the bound chunk storage')
                chunk, begin, end = b.ranges[p]
                state = self.state[p]
                if len(state) == 0:
                    flat_m, flat_v = b.moments(chunk)
                    state['step'] = 0
                    # per-tensor views of the flat moments, shaped like the optimizer's slice
                    state['exp_avg'] = flat_m[begin:end]
                    state['exp_avg_sq'] = flat_v[begin:end]
                entries.append((state, gi, b.chunk_index[chunk], begin, end))
        self._bound_entries = (signature, entries)
        return entries

    def _bound_hyper_indices(self, entries, hypers: Dict) -> List[int]:
        """Index of the hyper record of every bound entry -- the (group, step + 1) pair it will be
        updated with -- filling ``hypers`` on the way.  Host arithmetic only."""
        groups = self.param_groups
        seen: Dict = {}    # (group, step) -> hyper index: nearly always one step count per group
        idx_of = []
        for state, gi, _, _, _ in entries:
            k = (gi, state['step'])
            h = seen.get(k)
            if h is None:
                h = seen[k] = self._hyper_index(hypers, groups[gi], k[1] + 1)
            idx_of.append(h)
        return idx_of

    def hyper_table_of_next_step(self) -> np.ndarray:
        """The ElxHyper records the next step over the bound chunks would upload (a host array; nothing
        is launched or prepared): what a changed ``group['lr']`` turns into."""
        assert self._binding is not None, 'only for an optimizer bound to chunk storage'
        hypers: Dict = {}
        self._bound_hyper_indices(self._walk_bound(), hypers)
        return self._hyper_table(hypers)

    def _prepare_bound(self, hypers: Dict) -> Optional[_Prepared]:
        b = self._binding
        b.require_gpu()
        entries = self._walk_bound()
        if not entries:
            return None
        idx_of = self._bound_hyper_indices(entries, hypers)
        lowp_dtype = b.chunks[0].paired_chunk.chunk_dtype
        grad_code = dtype_code(lowp_dtype)
        lowp_code = _abi.ELX_NONE if b.zero_grads else grad_code
        device = b.launch_device()
        shard_ptrs = tuple(c.paired_chunk.shard.data_ptr() for c in b.chunks)
        key = ('bound', b.zero_grads, tuple(idx_of), shard_ptrs, tuple(c.shard.data_ptr() for c in b.chunks))

        def buffers():
            per_chunk: List[List[Tuple[int, int, int]]] = [[] for _ in b.chunks]
            for (state, gi, ci, begin, end), h in zip(entries, idx_of):
                per_chunk[ci].append((begin, end, h))
            out = []
            for i, c in enumerate(b.chunks):
                pc = c.paired_chunk
                assert pc.chunk_dtype == lowp_dtype, 'all parameter chunks of one optimizer share a dtype'
                flat_m, flat_v = b.moments(c)
                shard_ptr = 0 if b.zero_grads else pc.shard.data_ptr()
                out.append(FlatBuffer(grad=shard_ptr, lowp_out=shard_ptr, master=c.shard.data_ptr(),
                                      m=flat_m.data_ptr(), v=flat_v.data_ptr(), n_alloc=c.shard_size, n_valid=pc.n_valid,
                                      segs=sorted(per_chunk[i])))
            return out

        dplan = self._device_plan(key, buffers, lowp_dtype, grad_code, lowp_code, len(hypers), device,
                                  device_resident=all(c.shard.is_cuda and c.paired_chunk.shard.is_cuda for c in b.chunks))
        return _Prepared(dplan, self._hyper_table(hypers), grad_code, lowp_code, device, [e[0] for e in entries],
                         hypers.keys())

    # ---- standalone, on ordinary parameters

    def _watch_holds(self, watch) -> bool:
        """Whether every buffer a cached walk recorded is still the one in use: parameter, gradient (address and
        dtype) and, for a parameter that has stepped, its state entry with both moments where they were."""
        states = self.state
        for p, p_ptr, g_ptr, g_dtype, state, m_ptr, v_ptr in watch:
            g = p.grad
            if g is None:
                if g_ptr is not None:
                    return False
                continue
            if g_ptr is None or g.data_ptr() != g_ptr or g.dtype != g_dtype or p.data_ptr() != p_ptr:
                return False
            if states.get(p) is not state:
                return False
            m, v = state.get('exp_avg'), state.get('exp_avg_sq')
            if m is None or v is None or m.data_ptr() != m_ptr or v.data_ptr() != v_ptr:
                return False
        return True

    def _standalone_items(self):
        """(items, gradient dtype, device) of the parameters that carry a gradient: per parameter its state
        dict, its group index and (gradient, parameter, exp_avg, exp_avg_sq addresses, element count).  The
        walk with its checks is repeated only when a parameter, a gradient buffer, a state entry or one of its
        moments, or the group layout has changed since the last step (every buffer is watched by address, the
        gradient by dtype too)."""
        cache = self._standalone_cache
        if cache is not None:
            watch, layout, result = cache
            if layout == tuple(len(g['params']) for g in self.param_groups):
                if self._watch_holds(watch):
                    return result
        items, watch = [], []
        grad_dtype = None
        device = None
        for gi, group in enumerate(self.param_groups):
            for p in group['params']:
                if p.grad is None or p.numel() == 0:
                    watch.append((p, p.data_ptr(), None, None, None, 0, 0))
                    continue
                if p.device.type != 'cuda':
                    raise RuntimeError('HybridAdam runs on the GPU: parameters must live in device memory')
                if p.dtype != torch.float32:
                    raise TypeError('HybridAdam keeps fp32 parameters; low-precision training goes through '
                                    'ElixirOptimizer, which pairs them with fp32 master chunks')
                if not p.data.is_contiguous() or not p.grad.is_contiguous():
                    raise RuntimeError('HybridAdam needs contiguous parameters and gradients')
                if grad_dtype is None:
                    grad_dtype, device = p.grad.dtype, p.device
                elif p.grad.dtype != grad_dtype or p.device != device:
                    raise RuntimeError('all gradients of one step must share a dtype and a device')
                state = self.state[p]
                if len(state) == 0:
                    state['step'] = 0
                    state['exp_avg'] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state['exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.preserve_format)
                m_ptr, v_ptr = state['exp_avg'].data_ptr(), state['exp_avg_sq'].data_ptr()
                watch.append((p, p.data_ptr(), p.grad.data_ptr(), p.grad.dtype, state, m_ptr, v_ptr))
                items.append((state, gi, (p.grad.data_ptr(), p.data.data_ptr(), m_ptr, v_ptr, p.numel())))
        result = (items, grad_dtype, device)
        self._standalone_cache = (watch, tuple(len(g['params']) for g in self.param_groups), result)
        return result

    def _prepare_standalone(self, hypers: Dict) -> Optional[_Prepared]:
        items, grad_dtype, device = self._standalone_items()
        if not items:
            return None
        groups = self.param_groups
        seen: Dict = {}    # (group, step) -> hyper index
        idx_of = []
        for state, gi, _ in items:
            k = (gi, state['step'])
            h = seen.get(k)
            if h is None:
                h = seen[k] = self._hyper_index(hypers, groups[gi], k[1] + 1)
            idx_of.append(h)
        grad_code = dtype_code(grad_dtype)
        key = ('standalone', grad_code, tuple(it[2] for it in items), tuple(idx_of))

        def buffers():
            return [FlatBuffer(grad=g, lowp_out=0, master=p, m=m, v=v, n_alloc=n, n_valid=n, segs=[(0, n, h)])
                    for (_, _, (g, p, m, v, n)), h in zip(items, idx_of)]

        dplan = self._device_plan(key, buffers, grad_dtype, grad_code, _abi.ELX_NONE, len(hypers), device)
        return _Prepared(dplan, self._hyper_table(hypers), grad_code, _abi.ELX_NONE, device, [it[0] for it in items],
                         hypers.keys(), idx_of)


class FusedAdam(HybridAdam):
    """The device-only member of the reference's list of optimizers that take ``div_scale``
    (elixir/wrapper/optimizer.py:19: ``{FusedAdam, CPUAdam, HybridAdam}``).  Constructor and ``step``
    follow ColossalAI's ``FusedAdam`` as published (its source is not in the reference's tree):
    ``adamw_mode`` comes before ``weight_decay``, ``amsgrad`` is refused, ``set_grad_none`` is the
    default of ``zero_grad``; the legacy ``grads`` / ``output_params`` / ``scale`` / ``grad_norms``
    arguments of ``step`` are refused as they are there.  Same launches as ``HybridAdam``."""

    def __init__(self,
                 params,
                 lr: float = 1e-3,
                 bias_correction: bool = True,
                 betas: Tuple[float, float] = (0.9, 0.999),
                 eps: float = 1e-8,
                 adamw_mode: bool = True,
                 weight_decay: float = 0.,
                 amsgrad: bool = False,
                 set_grad_none: bool = True):
        if amsgrad:
            raise RuntimeError('FusedAdam does not support the AMSGrad variant.')
        super().__init__(params, lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay,
                         adamw_mode=adamw_mode)
        self.set_grad_none = set_grad_none

    def zero_grad(self, set_to_none: Optional[bool] = None):
        return super().zero_grad(set_to_none=self.set_grad_none if set_to_none is None else set_to_none)

    def step(self, closure=None, grads=None, output_params=None, scale=None, grad_norms=None, div_scale: float = -1,
             **kwargs):
        if any(p is not None for p in (grads, output_params, scale, grad_norms)):
            raise RuntimeError('FusedAdam has been updated.  Simply initialize it identically to torch.optim.Adam, and '
                               'call step() with no arguments.')
        return HybridAdam.step(self, closure, div_scale, **kwargs)

    step.hooked = True    # see HybridAdam.step


class CPUAdam(HybridAdam):
    """The host-side member of the same list: ColossalAI's ``CPUAdam(model_params, lr, bias_correction,
    betas, eps, weight_decay, adamw_mode, nvme_offload_fraction, nvme_offload_dir)`` with
    ``step(closure=None, div_scale=-1)`` -- the signature ``HybridAdam`` inherits there.  There is no CPU
    arithmetic in this package: chunk shards in pinned host memory are updated in place by the same
    launches over the host link, pageable host memory is refused."""
