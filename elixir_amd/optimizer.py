"""``ElixirOptimizer``: the optimizer wrapper of ``elixir/wrapper/optimizer.py`` with the same
constructor, methods and control flow, driving the HIP kernels.

One step is:

  1. one stats launch over every parameter chunk (overflow flag and sum of squares of the
     still-scaled gradients) -- none at all when the gradients arrived through the fused landing,
     which leaves the flags on the device;
  2. the decisions of optimizer.py:192-209 -- overflow -> skip and back off, otherwise combined scale
     = loss scale (x clip coefficient) -- taken ON THE DEVICE by the launch that folds the flags, in
     the float64 arithmetic of the reference's Python, and left where the update launch reads them;
     the decision and the 16 bytes of flags per chunk come back through pinned host memory for the
     host's bookkeeping (the reference pays two ``.item()`` per chunk at gradient-landing time, plus
     one for the loss scale, plus one for the norm);
  3. one fused launch, enqueued without waiting for 2.: unscale + Adam/AdamW on master/m/v +
     low-precision writeback (optimizer.py:216-219), which turns into the writeback alone when the
     decision says skip (optimizer.py:196-203).

With ``gated_step`` off, or when the flags of some chunks are already on the host, the host fetches the
flags, decides in Python floats and only then launches 3. (or the writeback alone).

Differences from the reference, all on purpose:
  * clipping works: ``max_norm > 0`` switches ``l2_norm_flag`` on for every parameter chunk (the
    reference never sets the flag and trips its own assertion, optimizer.py:152);
  * bfloat16 parameter chunks are accepted (``use_amp`` stays tied to float16, so bf16 trains
    with a constant scale of 1 and the overflow check still runs);
  * exp_avg / exp_avg_sq live in flat per-chunk buffers (``state[p]['exp_avg']`` are views);
  * ``state_dict`` / ``load_state_dict`` also carry the loss scaler, and loading copies into the
    flat buffers in place;
  * shards in pinned host memory are stepped by the same launches, in place over the host link.
"""
import logging
import math
import time
from collections import OrderedDict, defaultdict
from enum import Enum
from typing import Dict, List, Set, Tuple

import numpy as np
import torch
from torch.nn import Parameter

from . import _abi
from .chunk import (Chunk, DeviceTable, StatsArena, dtype_code, keep_grads_cached, kernel_device, launch_grad_stats,
                    read_grad_stats, resolve_pending_stats, stats_launch_blocks)
from .grad_scaler import BaseGradScaler, ConstantGradScaler, DynamicGradScaler
from .hybrid_adam import CPUAdam, FusedAdam, HybridAdam

_AVAIL_OPTIM_LIST = {FusedAdam, CPUAdam, HybridAdam}

# the one runtime signal of this path in the reference: optimizer.py:88 (a distributed logger) and :199
logger = logging.getLogger('elixir_amd.optimizer')


# What the wrapper and the inner optimizer bound to it read and call on a chunk object.  The first tuple is what
# the reference's wrapper uses of its own Chunk (optimizer.py:58-66,115-164,238-256; chunk.py:59-139); the second
# is what this build's step needs on top: where the flags of the gradients are kept between a landing launch and
# the step (a record slot in a device arena, fetched lazily), and the bookkeeping around it.
CHUNK_MEMBERS_OF_THE_REFERENCE = ('tensors_info', 'shard_begin', 'shard_size', 'shard', 'paired_chunk', 'overflow',
                                  'l2_norm', 'l2_norm_flag', 'optim_update', 'optim_sync_flag', 'torch_pg', 'is_replica',
                                  'chunk_dtype', 'shard_device', 'chunk_id')
CHUNK_MEMBERS_ADDED = ('n_valid', 'invalidate_stats', '_apply_stats', '_overflow', '_stats_fresh', '_stats_pending',
                       '_stats_slot', '_stats_pinned', '_stats_home', '_stats_event', '_stats_stream', '_take_stats_slot')


class OptimState(Enum):
    SCALED = 0
    UNSCALED = 1


def calc_combined_scale(loss_scale: float, total_norm, max_norm: float, clipping: bool) -> float:
    """optimizer.py:166-183 in Python floats: gradient = gradient / combined scale."""
    combined_scale = loss_scale
    if clipping:
        clip = ((total_norm / loss_scale) + 1e-6) / max_norm
        if clip > 1:
            combined_scale = clip * loss_scale
    if combined_scale == 1:
        return -1
    return combined_scale


class _EventPair:
    """Context manager that brackets launches with events on the current stream."""

    def __init__(self, sink, key):
        self.sink, self.key = sink, key

    def __enter__(self):
        if self.sink is not None:
            pair = self.sink.get(self.key)
            if pair is None:    # created once, recorded again every step: creating events is the costly part
                pair = self.sink[self.key] = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            self.begin, self.end = pair
            self.begin.record()
        return self

    def __exit__(self, *exc):
        if self.sink is not None:
            self.end.record()
        return False


class _DeviceStep:
    """Plumbing of a step that is decided on the device.

    What changes from step to step (loss scale, clipping threshold, the hyper records) is written into a
    control block in pinned host memory that the decision kernel reads; that kernel reports back into
    pinned host memory, the sequence number last, and the host polls it.  No launch of the step takes
    an argument that changes, so the launches can be recorded once as a HIP graph and replayed."""

    POLL_LIMIT_S = 0.05    # then the stream is synchronised instead (the report has arrived by then)
    MAX_GRAPHS = 4

    def __init__(self, device: torch.device, n_chunks: int):
        self.device, self.n_chunks = device, n_chunks
        self.max_hypers = _abi.max_ctl_hypers()
        ctl_head, rep_head = _abi.STEP_CTL_DTYPE.itemsize, _abi.STEP_REPORT_DTYPE.itemsize
        hyp, rec = _abi.HYPER_DTYPE.itemsize, _abi.STATS_DTYPE.itemsize
        self.ctl = torch.zeros(ctl_head + self.max_hypers * hyp, dtype=torch.uint8, pin_memory=True)
        self.report = torch.zeros(rep_head + n_chunks * rec, dtype=torch.uint8, pin_memory=True)
        self._ctl_bytes = self.ctl.numpy()
        self._ctl_head = self._ctl_bytes[:ctl_head].view(_abi.STEP_CTL_DTYPE)
        report_bytes = self.report.numpy()
        self.report_head = report_bytes[:rep_head].view(_abi.STEP_REPORT_DTYPE)
        self.report_stats = report_bytes[rep_head:].view(_abi.STATS_DTYPE)
        # device side: hyper table of the update launch | decision | counter | per-chunk records
        self.dev = torch.zeros(self.max_hypers * hyp + 64 + n_chunks * rec, dtype=torch.uint8, device=device)
        base = self.dev.data_ptr()
        self.d_hypers = base
        self.d_decision = base + self.max_hypers * hyp
        self.d_counter = self.d_decision + 32
        self.d_stats = self.d_decision + 64
        self.seq = 0
        self.partials = None             # workspace of the stats launch
        self.seen = set()                # launch sequences that have run once (eagerly)
        self.graphs: Dict = {}           # launch sequence -> (graph, objects its launches point into)

    def write_ctl(self, loss_scale: float, max_norm: float, clipping: bool, hyper_host: np.ndarray) -> int:
        self.seq += 1
        n = len(hyper_host)
        head = self._ctl_head
        at = head.itemsize
        self._ctl_bytes[at:at + hyper_host.nbytes] = hyper_host.view(np.uint8).reshape(-1)
        head[0] = (loss_scale, max_norm, int(clipping), n, self.seq)
        return self.seq

    def partials_buffer(self, records: int) -> int:
        need = records * _abi.STATS_DTYPE.itemsize
        if self.partials is None or self.partials.numel() < need:
            self.partials = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self.partials.data_ptr()

    def wait_report(self, seq: int, stream: torch.cuda.Stream):
        """Polls the sequence number of the report; returns (decision record, per-chunk records)."""
        head = self.report_head
        give_up = time.perf_counter() + self.POLL_LIMIT_S
        while int(head['seq'][0]) != seq:
            if time.perf_counter() > give_up:
                stream.synchronize()
                if int(head['seq'][0]) != seq:
                    raise RuntimeError('the decision kernel has run but its report did not arrive in host memory')
                break
        if int(head['status'][0]) != 0:
            raise RuntimeError(f'the decision kernel refused its control block (status {int(head["status"][0])})')
        return head[0], self.report_stats


class ElixirOptimizer(torch.optim.Optimizer):
    """A wrapper for optimizers; one ElixirOptimizer corresponds to one chunked module.

    Like the reference's wrapper (optimizer.py:27, a ``ColossalaiOptimizer``) it IS a
    ``torch.optim.Optimizer`` -- learning-rate schedulers and anything else that checks the type accept
    it -- without running ``Optimizer.__init__``: ``param_groups``, ``state`` and ``defaults`` are those
    of the inner optimizer, so a scheduler that edits ``group['lr']`` edits what the next step uploads.

    Args:
        module: the chunked module (``param_chunk_group``, ``optim_chunk_group``,
            ``fetcher.get_one_chunk``, ``use_amp``)
        optimizer: the inner optimizer built on the module's real parameters; a ``HybridAdam``
            takes the fused path, any other element-wise torch optimizer runs unfused and only
            without loss scaling and clipping (optimizer.py:211-214)
        initial_scale ... max_scale: dynamic loss scale settings (used when ``module.use_amp``)
        max_norm: global L2 gradient-norm clip, 0 disables
    """

    def __init__(self,
                 module,
                 optimizer: torch.optim.Optimizer,
                 initial_scale: float = 32768,
                 min_scale: float = 1,
                 growth_factor: float = 2,
                 backoff_factor: float = 0.5,
                 growth_interval: int = 1000,
                 hysteresis: int = 2,
                 max_scale: float = 2**24,
                 max_norm: float = 0.0,
                 norm_type: float = 2.0,
                 init_step=False):
        self.optim = optimizer
        # Optimizer.__init__ is not run (the groups, the state and the defaults are the inner optimizer's), so
        # what it would have set up for hooks registered on THIS object is set up here; step() dispatches them
        self._optimizer_step_pre_hooks = OrderedDict()
        self._optimizer_step_post_hooks = OrderedDict()
        for attr in ('param_chunk_group', 'optim_chunk_group', 'fetcher', 'use_amp'):
            assert hasattr(module, attr), f'module lacks {attr}: it is not a chunked module'
        self.scaled_optimizer = False
        if type(optimizer) in _AVAIL_OPTIM_LIST:
            self.scaled_optimizer = True

        self.module = module
        self.param_chunk_group = module.param_chunk_group
        self.optim_chunk_group = module.optim_chunk_group

        self.optim_state = OptimState.UNSCALED
        self.param_to_range: Dict[Parameter, Tuple[int, int]] = dict()
        self.param_to_optim_chunk: Dict[Parameter, Chunk] = dict()
        self.param_chunk_set: Set[Chunk] = self.param_chunk_group.fused_chunks.union(
            self.param_chunk_group.float_chunks)
        self._param_chunk_list: List[Chunk] = sorted(self.param_chunk_set)
        # Every parameter chunk gets its record slot in the device arena now, in chunk order: landings then
        # leave the flags side by side whatever order the chunks land in (backward lands the last chunk
        # first, one launch per chunk), and the step folds them with one launch, without a host read.
        shards = [c.shard for c in self._param_chunk_list]
        if shards and all(t.is_cuda and t.device == shards[0].device for t in shards):
            StatsArena.get(shards[0].device).pin(self._param_chunk_list)

        self.clipping_flag = max_norm > 0.0
        self.max_norm = max_norm
        if self.clipping_flag:
            assert norm_type == 2.0, 'ElixirOptimizer only supports L2 norm now'
            for param_chunk in self.param_chunk_set:
                param_chunk.l2_norm_flag = True

        self.__init__optimizer()

        # Grad scaler
        self.grad_scaler: BaseGradScaler = None
        if module.use_amp:
            self.grad_scaler = DynamicGradScaler(initial_scale=initial_scale,
                                                 min_scale=min_scale,
                                                 growth_factor=growth_factor,
                                                 backoff_factor=backoff_factor,
                                                 growth_interval=growth_interval,
                                                 hysteresis=hysteresis,
                                                 max_scale=max_scale)
        else:
            self.grad_scaler = ConstantGradScaler(1.0, verbose=False)

        self._binding = None
        if self.scaled_optimizer:
            ranges = {
                fake: (self.param_to_optim_chunk[fake], ) + self.param_to_range[fake] for fake in self.param_to_range
            }
            if ranges:
                self._binding = self.optim.bind_chunks(ranges)
        self._stats_table = None
        self._all_stats_table = None
        self._stats_workspace: Dict = {}
        # the step decided on the device (no wait between the flags and the update); False: the host
        # fetches the flags, decides and only then launches
        self.gated_step = True
        # with gated_step: record the launches of a step once as a HIP graph and replay it (the first step
        # over a set of tables runs eagerly, the second records; nothing is recorded while kernel_events is set)
        self.graph_step = False
        self._device_step: _DeviceStep = None
        # most hyper records a step decided on the device can carry (the control block's capacity); a step
        # with more is decided on the host, from the same single pass over the gradients
        self.max_device_hypers = _abi.max_ctl_hypers()
        self._wb_table = None
        self.last_step_info: Dict = {}
        # when set to a dict, step() records (begin, end) torch.cuda.Event pairs on the launch
        # stream under the keys 'stats' and 'update' (for per-kernel timing by a benchmark)
        self.kernel_events = None
        # cap on resident update workgroups per compute unit (0 = the library default)
        self.blocks_per_cu = 0

        if init_step:
            # allocate memory before training
            self.__zero_step()

    # ------------------------------------------------------------------ torch.optim.Optimizer through the inner optimizer

    @property
    def param_groups(self):
        return self.optim.param_groups

    @param_groups.setter
    def param_groups(self, value):
        self.optim.param_groups = value

    @property
    def defaults(self):
        return self.optim.defaults

    @defaults.setter
    def defaults(self, value):
        self.optim.defaults = value

    @property
    def state(self):
        return self.optim.state

    @state.setter
    def state(self, value):
        self.optim.state = value

    def __repr__(self):
        return f'{type(self).__name__}({self.optim!r})'

    def add_param_group(self, *args, **kwargs):
        return self.optim.add_param_group(*args, **kwargs)

    # hooks around state_dict / load_state_dict belong to the optimizer that produces and takes the state
    def register_state_dict_pre_hook(self, *args, **kwargs):
        return self.optim.register_state_dict_pre_hook(*args, **kwargs)

    def register_state_dict_post_hook(self, *args, **kwargs):
        return self.optim.register_state_dict_post_hook(*args, **kwargs)

    def register_load_state_dict_pre_hook(self, *args, **kwargs):
        return self.optim.register_load_state_dict_pre_hook(*args, **kwargs)

    def register_load_state_dict_post_hook(self, *args, **kwargs):
        return self.optim.register_load_state_dict_post_hook(*args, **kwargs)

    def __getstate__(self):
        raise TypeError('an ElixirOptimizer is tied to the chunk storage of its module and cannot be copied or '
                        'pickled: save state_dict() and load it into a newly built one')

    def __deepcopy__(self, memo):
        self.__getstate__()

    def state_dict(self):
        """The inner optimizer's state in torch's packed layout (step, exp_avg, exp_avg_sq per fake
        parameter -- the slice of each tensor this process owns -- and the group hyper-parameters),
        plus the loss scaler under ``grad_scaler``.  The reference forwards to the inner optimizer
        and loses the scaler; resuming a mixed-precision run needs both."""
        packed = self.optim.state_dict()
        packed['grad_scaler'] = self.grad_scaler.state_dict()
        return packed

    def load_state_dict(self, state_dict, *args, **kwargs):
        state_dict = dict(state_dict)
        scaler_state = state_dict.pop('grad_scaler', None)
        ret = self.optim.load_state_dict(state_dict, *args, **kwargs)
        if scaler_state is not None:
            self.grad_scaler.load_state_dict(scaler_state)
        return ret

    # ------------------------------------------------------------------ set-up

    def __init__optimizer(self):
        """optimizer.py:238-265: every real parameter becomes a zero-size fake parameter that
        stands for its slice of this process's shard; group hyper-parameters are untouched."""

        def get_range_pair(local_chunk: Chunk, local_param: Parameter):
            param_info = local_chunk.tensors_info[local_param]
            begin = max(0, param_info.offset - local_chunk.shard_begin)
            end = min(local_chunk.shard_size, param_info.end - local_chunk.shard_begin)
            return begin, end

        for group in self.param_groups:
            fake_params_list = list()

            for param in group['params']:
                if not param.requires_grad:
                    continue

                param_chunk = self.module.fetcher.get_one_chunk(param)
                range_pair = get_range_pair(param_chunk, param)
                if range_pair[0] >= range_pair[1]:
                    continue

                grad_device = param_chunk.shard.device
                fake_param = torch.nn.Parameter(torch.empty([0], device=grad_device))
                self.param_to_optim_chunk[fake_param] = param_chunk.paired_chunk
                self.param_to_range[fake_param] = range_pair

                fake_params_list.append(fake_param)

            group['params'] = fake_params_list

    def __zero_step(self):
        """optimizer.py:94-113: one inner step with zero gradients, so that the optimizer state
        exists before training.  It counts as a step (state['step'] becomes 1) and, with decoupled
        weight decay, decays the master weights once; the low-precision copy is not refreshed."""
        if self._binding is not None:
            self._binding.zero_grads = True
            try:
                self.optim.step()
            finally:
                self._binding.zero_grads = False
                self._binding.fused_writeback = False
        else:
            for group in self.param_groups:
                for fake_param in group['params']:
                    optim_chunk = self.param_to_optim_chunk[fake_param]
                    begin, end = self.param_to_range[fake_param]
                    fake_param.data = optim_chunk.shard[begin:end]
                    fake_param.grad = torch.zeros_like(fake_param.data)
            self.optim.step()
        self.zero_grad()
        self._update_fp16_params(update_flag=False)

    # ------------------------------------------------------------------ pieces of the step

    def _set_grad_ptr(self):
        """optimizer.py:115-124.  A bound HybridAdam reads gradients and master weights straight
        from the chunk buffers, so nothing needs to be pointed anywhere."""
        if self._binding is not None:
            return
        for group in self.param_groups:
            for fake_param in group['params']:
                optim_chunk = self.param_to_optim_chunk[fake_param]
                begin, end = self.param_to_range[fake_param]
                param_chunk = optim_chunk.paired_chunk

                fake_param.data = param_chunk.shard[begin:end]
                fake_param.grad = fake_param.data
                fake_param.data = optim_chunk.shard[begin:end]

    def _update_fp16_params(self, update_flag: bool = True):
        """optimizer.py:126-135: detach the fake parameters and refresh the low-precision shards
        from the fp32 shards -- unless the fused launch has just done so."""
        if self._binding is None:
            none_tensor = torch.empty([0])
            for group in self.param_groups:
                for fake_param in group['params']:
                    assert fake_param.grad is None
                    fake_param.data = none_tensor.to(fake_param.device)

        if not update_flag:
            return
        if hasattr(self.module, 'mark_params_stale'):
            self.module.mark_params_stale()    # the next forward pass reads the refreshed shards
        if self._binding is not None and self._binding.fused_writeback:
            self._binding.fused_writeback = False
            for param_chunk in self.param_chunk_set:
                param_chunk.optim_sync_flag = True
            return
        self._writeback_all()

    def _writeback_all(self) -> None:
        """``optim_update`` for every parameter chunk in one launch."""
        gpu_chunks = [c for c in self._param_chunk_list if c.shard_device.type == 'cuda']
        for c in self._param_chunk_list:
            if c.shard_device.type != 'cuda':
                c.optim_update()
        if not gpu_chunks:
            return
        key = tuple((c.shard.data_ptr(), c.paired_chunk.shard.data_ptr()) for c in gpu_chunks)
        if self._wb_table is None or self._wb_table[0] != key:
            tile = _abi.tile_elems()
            rows = np.zeros(len(gpu_chunks), dtype=_abi.CHUNK_DTYPE)
            tiles = 0
            for i, c in enumerate(gpu_chunks):
                friend = c.paired_chunk
                assert friend is not None and not friend.is_replica
                assert friend.shard_device == c.shard_device
                rows[i]['lowp_out'] = c.shard.data_ptr()
                rows[i]['master'] = friend.shard.data_ptr()
                rows[i]['m'] = friend.shard.data_ptr()
                rows[i]['v'] = friend.shard.data_ptr()
                rows[i]['n_alloc'] = c.shard_size
                rows[i]['n_valid'] = c.n_valid
                rows[i]['tile_begin'] = tiles
                tiles += (c.shard_size + tile - 1) // tile
            code = dtype_code(gpu_chunks[0].chunk_dtype)
            info = _abi.check_tables(rows, None, 0, code, code)
            self._wb_table = (key, DeviceTable(rows, gpu_chunks[0].shard_device), info, code,
                              max(c.shard_size for c in gpu_chunks))
        _, table, info, code, max_elems = self._wb_table
        stream = torch.cuda.current_stream(table.dev.device).cuda_stream
        _abi.writeback_mt(table.ptr, len(table), code, max_elems, info.aligned, stream)
        for c in gpu_chunks:
            c.optim_sync_flag = True

    def _launch_chunk_stats(self):
        """Enqueues the flags pass for every parameter chunk whose gradients landed without them:
        one launch over the chunk list.  Returns what ``_collect_chunk_stats`` needs."""
        pending = [c for c in self._param_chunk_list if not c._stats_fresh and not c._stats_pending]
        if not pending:
            return None
        device = kernel_device(c.shard for c in pending)
        ids = tuple((c.chunk_id, c.shard.data_ptr()) for c in pending)    # the table holds addresses
        if self._stats_table is None or self._stats_table[0] != ids:
            rows = np.zeros(len(pending), dtype=_abi.CHUNK_DTYPE)
            for i, c in enumerate(pending):
                rows[i]['grad'] = c.shard.data_ptr()
                rows[i]['n_alloc'] = c.shard_size
                rows[i]['n_valid'] = c.n_valid
            self._stats_table = (ids, rows, DeviceTable(rows, device))
        _, rows, table = self._stats_table
        with self._timed('stats'):
            records = launch_grad_stats(rows, dtype_code(pending[0].chunk_dtype), device, table=table,
                                        workspace=self._stats_workspace)
        return pending, records

    def _collect_chunk_stats(self, launched) -> None:
        """One device-to-host copy of 16 bytes per chunk: the only wait of the step."""
        resolve_pending_stats(self._param_chunk_list)    # records left behind by fused landings
        if launched is None:
            return
        pending, records = launched
        stats = read_grad_stats(records)
        for c, rec in zip(pending, stats):
            c._apply_stats(bool(rec['overflow']), float(rec['sumsq']))

    def _refresh_chunk_stats(self) -> None:
        self._collect_chunk_stats(self._launch_chunk_stats())

    def _timed(self, key: str):
        return _EventPair(self.kernel_events, key)

    def _check_overflow(self) -> bool:
        # calculate the overflow counter
        overflow_counter = 0
        for param_chunk in self.param_chunk_set:
            overflow_counter += int(param_chunk.overflow)
        return overflow_counter > 0

    def _clear_optim_states(self) -> None:
        for param_chunk in self.param_chunk_set:
            param_chunk.invalidate_stats()

    def _calc_global_norm(self) -> float:
        """optimizer.py:149-164 on one process: the per-group sum passes through a one-element fp32
        buffer before the square root."""
        group_to_norm = defaultdict(float)
        for param_chunk in self._param_chunk_list:    # a fixed order: float64 sums depend on it
            assert param_chunk.l2_norm is not None
            assert not param_chunk.is_replica
            group_to_norm[param_chunk.torch_pg] += param_chunk.l2_norm

        norm_sqr = 0.0
        for group, part_norm in group_to_norm.items():
            norm_sqr += float(np.float32(part_norm))

        global_norm = math.sqrt(norm_sqr)
        return global_norm

    def _get_combined_scale(self):
        assert self.optim_state == OptimState.SCALED
        loss_scale = self.loss_scale
        self.optim_state = OptimState.UNSCALED

        total_norm = self._calc_global_norm() if self.clipping_flag else None
        self.last_step_info['total_norm'] = total_norm
        return calc_combined_scale(loss_scale, total_norm, self.max_norm, self.clipping_flag)

    @property
    def loss_scale(self):
        return self.grad_scaler.scale_value

    def zero_grad(self, *args, **kwargs):
        if self._binding is not None:
            return None    # bound fake parameters never carry a .grad: nothing to drop
        return self.optim.zero_grad(set_to_none=True)

    # ------------------------------------------------------------------ the step, decided on the device

    def _stats_source(self):
        """Where the decision kernel finds the flags of ALL parameter chunks, or None when they are not
        all in one place: ('launch', None) -- no chunk has flags, one stats launch over all of them is
        needed -- or ('arena', first slot) -- fused landings left every chunk's record in consecutive
        slots of the device arena."""
        chunks = self._param_chunk_list
        if not chunks:
            return None
        if all(not c._stats_fresh and not c._stats_pending for c in chunks):
            return ('launch', None)
        if all(c._stats_pending for c in chunks):
            first = chunks[0]._stats_slot
            if all(c._stats_slot == first + i for i, c in enumerate(chunks)):
                return ('arena', first)
        return None

    def _all_chunks_stats_table(self, device: torch.device):
        chunks = self._param_chunk_list
        ids = tuple(c.chunk_id for c in chunks)
        ptrs = tuple(c.shard.data_ptr() for c in chunks)
        if self._all_stats_table is None or self._all_stats_table[0] != (ids, ptrs):
            # checked once per set of buffers, BEFORE anything is launched on them: a shard in pageable host
            # memory is refused here (a launch over it would fault the device)
            kernel_device(c.shard for c in chunks)
            rows = np.zeros(len(chunks), dtype=_abi.CHUNK_DTYPE)
            for i, c in enumerate(chunks):
                rows[i]['grad'] = c.shard.data_ptr()
                rows[i]['n_alloc'] = c.shard_size
                rows[i]['n_valid'] = c.n_valid
            cached = (all(c.shard.is_cuda for c in chunks)
                      and keep_grads_cached(rows, dtype_code(chunks[0].chunk_dtype)))
            self._all_stats_table = ((ids, ptrs), DeviceTable(rows, device),
                                     stats_launch_blocks(int(rows['n_valid'].max()), len(chunks), cached),
                                     bool(np.all(rows['grad'] % 16 == 0)), cached)
        return self._all_stats_table[1:]

    def _step_on_device(self, source) -> bool:
        """The step without a wait between the flags and the update: the decisions of
        optimizer.py:137-183 are taken by the kernel that folds the flags, which leaves them in the hyper
        table of the update launch; the update is enqueued right behind it and reads them there (on a skip
        it only refreshes the low-precision copies).  The decision and the flags come back through pinned
        host memory while the update runs, for the host's bookkeeping (scaler, step counts, chunk flags).
        Returns False when nothing was prepared to launch this way."""
        inner = self.optim
        chunks = self._param_chunk_list
        n = len(chunks)
        device = self._binding.launch_device()
        eng = self._device_step
        if eng is None or eng.device != device or eng.n_chunks != n:
            eng = self._device_step = _DeviceStep(device, n)
        main = torch.cuda.current_stream(device)
        kind, first_slot = source
        early = False
        if kind == 'launch':
            table, bpc, aligned, cached = self._all_chunks_stats_table(device)
            partials = eng.partials_buffer(n * bpc)
            stats_args = (table.ptr, n, dtype_code(chunks[0].chunk_dtype), bpc, partials, not aligned)
            keep = (table, eng.partials)
            if not self.graph_step and self.kernel_events is None:
                # the stats launch needs nothing of what follows: it goes out first, and the host prepares
                # the rest of the step (tables, control block) while the device reads the gradients
                _abi.grad_partials_mt(*stats_args, main.cuda_stream, keep_cached=cached)
                early = True
        else:
            arena = StatsArena.get(chunks[0].shard_device)
            for event in {c._stats_event for c in chunks
                          if c._stats_event is not None and c._stats_stream != main.cuda_stream}:
                main.wait_event(event)    # landings that ran on another stream
            bpc, partials, stats_args, keep, cached = 1, arena.ptr(first_slot), None, (arena, ), False
        inner.prepare_step(upload=False)
        prep = inner._prepared
        if prep is None or prep.dplan.rows is None or len(prep.hyper_host) > min(self.max_device_hypers, eng.max_hypers):
            if early:
                # The gradients have been read already: the partials are folded by the same launch, with a
                # control block that carries no hyper records, and its report brings every chunk's flags to
                # the host, which decides.  The gradients are not read a second time.
                seq = eng.write_ctl(float(self.loss_scale), float(self.max_norm) if self.clipping_flag else 1.0,
                                    self.clipping_flag, np.zeros(0, dtype=_abi.HYPER_DTYPE))
                _abi.finish_decide(partials, n, bpc, eng.d_stats, eng.ctl.data_ptr(), eng.d_hypers, eng.max_hypers,
                                   eng.d_decision, eng.report.data_ptr(), eng.d_counter, main.cuda_stream)
                _, stats = eng.wait_report(seq, main)
                for c, r in zip(chunks, stats):
                    c._apply_stats(bool(r['overflow']), float(r['sumsq']))
            return False
        assert prep.device == device
        # the control block is complete before the launch that reads it is issued
        seq = eng.write_ctl(float(self.loss_scale), float(self.max_norm), self.clipping_flag, prep.hyper_host)
        prep.d_hypers = eng.d_hypers

        def enqueue():
            stream = torch.cuda.current_stream(device).cuda_stream
            with self._timed('stats' if stats_args is not None else 'decide'):
                if stats_args is not None and not early:
                    _abi.grad_partials_mt(*stats_args, stream, keep_cached=cached)
                # the decision launch also arms the row table of the update launch: no valid element in any row
                # when the step is skipped (the update then only refreshes), every row's own count otherwise
                _abi.finish_decide(partials, n, bpc, eng.d_stats, eng.ctl.data_ptr(), eng.d_hypers, eng.max_hypers,
                                   eng.d_decision, eng.report.data_ptr(), eng.d_counter, stream,
                                   d_rows=prep.dplan.rows.ptr, d_gated_rows=prep.dplan.gated_rows.ptr,
                                   n_rows=len(prep.dplan.plan.rows), d_armed=prep.dplan.armed.data_ptr())
            with self._timed('update'):
                # through step(): the inner optimizer's hooks fire
                inner.step(gated=True, defer_commit=True, armed_rows=True)

        timing = self.kernel_events is not None or inner.kernel_events is not None
        key = (id(prep.dplan), kind, partials, bpc, inner.blocks_per_cu, stats_args[0] if stats_args else 0)
        if self.graph_step and not timing and key in eng.graphs:
            inner.adopt_prepared()
            eng.graphs[key][0].replay()
        elif self.graph_step and not timing and key in eng.seen:
            if len(eng.graphs) >= eng.MAX_GRAPHS:
                eng.graphs.clear()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, capture_error_mode='thread_local'):
                enqueue()
            eng.graphs[key] = (graph, prep.dplan, keep)    # what the recorded launches point into stays alive
            graph.replay()
        else:
            eng.seen.add(key)
            enqueue()

        device_says, stats = eng.wait_report(seq, main)
        for c, r in zip(chunks, stats):
            c._stats_pending = False
            c._stats_event = None
            c._apply_stats(bool(r['overflow']), float(r['sumsq']))

        # what the device decided is what happened: the host records it
        found_inf = bool(device_says['skip'])
        assert found_inf == self._check_overflow()
        self.last_step_info = dict(found_inf=found_inf, combined_scale=None, total_norm=None,
                                   chunk_overflow=[c._overflow for c in chunks])
        self.optim_state = OptimState.UNSCALED
        if found_inf:
            logger.info('Found overflow. Skip step')
            inner.abort_step()
        else:
            inner.commit_step()
            combined_scale = float(device_says['combined_scale'])
            self.last_step_info['combined_scale'] = -1 if combined_scale == -1.0 else combined_scale
            if self.clipping_flag:
                self.last_step_info['total_norm'] = float(device_says['total_norm'])
        self.grad_scaler.update(found_inf)
        self._clear_optim_states()
        self.zero_grad()
        self._update_fp16_params()
        return True

    # ------------------------------------------------------------------ the step

    def step(self, *args, **kwargs):
        """optimizer.py:185-220.  Step hooks registered on this object (``register_step_pre_hook`` /
        ``register_step_post_hook``) run around it.  torch's process-wide step hooks are not run here: as with
        the reference's wrapper they fire in the inner optimizer's own ``step``, once per step, with the inner
        optimizer as their argument (a step decided on the device has issued that call before it knows
        whether the step is skipped, so they also fire on a skipped step)."""
        if not (self._optimizer_step_pre_hooks or self._optimizer_step_post_hooks):
            return self._step(*args, **kwargs)
        for hook in list(self._optimizer_step_pre_hooks.values()):
            result = hook(self, args, kwargs)
            if result is not None:
                if not (isinstance(result, tuple) and len(result) == 2):
                    raise RuntimeError(f'{hook} must return None or a tuple of (new_args, new_kwargs), but got {result}.')
                args, kwargs = result
        out = self._step(*args, **kwargs)
        for hook in list(self._optimizer_step_post_hooks.values()):
            hook(self, args, kwargs)
        return out

    def _step(self, *args, **kwargs):
        if (self.gated_step and self._binding is not None and self.scaled_optimizer and not args and not kwargs
                and not self._binding.zero_grads and self.optim_state == OptimState.SCALED):
            source = self._stats_source()
            if source is not None:
                self._set_grad_ptr()
                if self._step_on_device(source):
                    return None
        launched = self._launch_chunk_stats()
        if self._binding is not None and not args and not kwargs:
            # host work of the update launch, done while the flags pass runs on the device
            self.optim.prepare_step()
        self._collect_chunk_stats(launched)
        self._set_grad_ptr()
        found_inf = self._check_overflow()
        self.last_step_info = dict(found_inf=found_inf, combined_scale=None, total_norm=None,
                                   chunk_overflow=[c._overflow for c in self._param_chunk_list])

        if found_inf:
            logger.info('Found overflow. Skip step')
            if self._binding is not None:
                self.optim.discard_prepared()
            self.optim_state = OptimState.UNSCALED    # no need to unscale grad
            self.grad_scaler.update(found_inf)    # update gradient scaler
            self._clear_optim_states()    # clear chunk states used for optimizer update
            self.zero_grad()    # reset all gradients
            self._update_fp16_params()
            return

        # get combined scale. combined scale = loss scale * clipping norm
        # so that gradient = gradient / combined scale
        combined_scale = self._get_combined_scale()

        # the launch goes out first; the bookkeeping that does not feed it follows while it runs
        if not self.scaled_optimizer:
            assert combined_scale == -1, 'You should use an optimizer in the available list:\n' \
            f'{_AVAIL_OPTIM_LIST}'
            ret = self.optim.step(*args, **kwargs)
        else:
            with self._timed('update'):
                ret = self.optim.step(div_scale=combined_scale, *args, **kwargs)

        self.last_step_info['combined_scale'] = combined_scale
        self.grad_scaler.update(found_inf)
        self._clear_optim_states()
        self.zero_grad()
        self._update_fp16_params()
        return ret

    def clip_grad_norm(self, model: torch.nn.Module, max_norm: float, norm_type: float = 2.0):
        raise NotImplementedError

    def backward(self, loss: torch.Tensor):
        loss = self.loss_scale * loss
        self.optim_state = OptimState.SCALED
        self.module.backward(loss)
        self.prepare_ahead()

    def prepare_ahead(self) -> None:
        """Builds and uploads the tables of the coming step now, while the device is still busy with
        backward and the landing of the gradients; ``step()`` then finds them ready (and rebuilds them
        if a hyper-parameter has changed in between)."""
        if self._binding is not None:
            try:
                # a step decided on the device hands the hyper records over in its control block
                self.optim.prepare_step(upload=not self.gated_step)
            except RuntimeError:
                self.optim.discard_prepared()    # nothing to prepare for: step() is where the refusal belongs

    def backward_by_grad(self, tensor: torch.Tensor, grad: torch.Tensor):
        self.optim_state = OptimState.SCALED
        self.module.backward_by_grad(tensor, grad)
        self.prepare_ahead()

    def mark_gradients_scaled(self) -> None:
        """For callers that land gradients in the chunk shards themselves (no ``backward`` through
        this wrapper): declares that the shards now hold gradients scaled by ``loss_scale`` and, as
        ``backward`` does at this point, prepares the tables of the coming step."""
        self.optim_state = OptimState.SCALED
        self.prepare_ahead()
