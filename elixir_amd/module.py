"""The module side of the optimizer step: chunk plans and the pairing of low-precision parameter
chunks with fp32 optimizer chunks (``elixir/search/result.py``, ``elixir/search/mini_waste.py:78-96``,
``elixir/wrapper/module.py:21-25,77-138,258-344``).

``ElixirModule`` here is the part of the reference's module wrapper that ``ElixirOptimizer`` reads:
it builds the paired chunk groups and exposes ``param_chunk_group``, ``optim_chunk_group``,
``fetcher.get_one_chunk``, ``use_amp``, ``state_dict`` / ``load_state_dict``.  The hook-driven
forward/backward (replicated cache, gather, reduce-scatter) is not part of this path; in its place
``land_gradients`` moves the ``.grad`` of the wrapped module's parameters into the chunk shards the
way the reference's gradient handler and chunk reduction leave them, and ``materialize_params``
points the parameters back at the refreshed low-precision values.
"""
from collections import OrderedDict
from typing import Any, Dict, Iterable, List, Mapping, NamedTuple, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .chunk import Chunk, ChunkGroup, gpu_device, land_tensors


class ChunkPlan(NamedTuple):
    """Instructs the initialization of a chunk (result.py:8-20)."""
    name_list: List[str]
    chunk_size: int
    chunk_dtype: torch.dtype
    kwargs: Dict


class SearchResult(object):

    def __init__(self, chunk_group: ChunkGroup, chunk_plans: List[ChunkPlan],
                 param_called_per_step: List[List[str]] = None) -> None:
        super().__init__()
        self.chunk_group = chunk_group
        self.param_chunk_plans = chunk_plans
        self.param_called_per_step = param_called_per_step


def to_divide(a: int, b: int) -> int:
    return a + (-a % b)


def greedy_groups(sizes: Sequence[int], chunk_size: int) -> List[List[int]]:
    """The packing rule of mini_waste.py:78-96: walk the tensors in order and open a new chunk
    whenever the room left in the current one is smaller than the next tensor.  (A tensor without elements
    at the head of the list opens the first chunk here; the reference files it under its last one.)"""
    groups: List[List[int]] = []
    last_left = 0
    for i, p_size in enumerate(sizes):
        if last_left < p_size or not groups:
            last_left = chunk_size
            groups.append([])
        assert last_left >= p_size, f'tensor {i} with {p_size} elements does not fit a chunk of {chunk_size}'
        last_left -= p_size
        groups[-1].append(i)
    return groups


def greedy_search(named_sizes: Sequence[Tuple[str, int]], chunk_size: int, dtype: torch.dtype,
                  shard_device: Optional[torch.device] = None) -> SearchResult:
    """A search result that packs every tensor into public chunks of one size with the greedy rule."""
    names = [n for n, _ in named_sizes]
    groups = greedy_groups([s for _, s in named_sizes], chunk_size)
    kwargs = {} if shard_device is None else dict(shard_device=shard_device)
    plans = [ChunkPlan([names[i] for i in g], chunk_size, dtype, dict(kwargs)) for g in groups]
    return SearchResult(ChunkGroup(None), plans)


def simple_groups(sizes: Sequence[int], split_number: int) -> Tuple[List[List[int]], int]:
    """The split rule of search/simple.py:30-74: the tensors, in order, are cut into
    ``min(len, split_number)`` runs by COUNT (the first ``len % split_number`` runs hold one tensor more);
    every public chunk gets the size of the fullest run.  Returns (groups of indices, that size)."""
    n = len(sizes)
    split_number = min(n, split_number)
    if split_number <= 0:
        return [], 0
    average, left = divmod(n, split_number)
    groups, at = [], 0
    for i in range(split_number):
        count = average + (1 if i < left else 0)
        groups.append(list(range(at, at + count)))
        at += count
    return groups, max(sum(sizes[i] for i in g) for g in groups)


def simple_search(named_sizes: Sequence[Tuple[str, int]], group_size: int, split_number: int, dtype: torch.dtype,
                  private_names: Sequence[str] = (), shard_device: Optional[torch.device] = None) -> SearchResult:
    """The chunk plans of the reference's ``simple_search`` (search/simple.py:77-110, search/base.py:87-108)
    for a tensor list given by name and size: every tensor named in ``private_names`` (the parameters a
    model uses more than once, search/utils.py:24-33) gets a private chunk of its own size rounded up
    to ``group_size``, marked ``rcache_fused``; the others are split by ``simple_groups`` into public
    chunks of one size (rounded up to ``group_size``).  Private plans come first."""
    private = set(private_names)
    kwargs = {} if shard_device is None else dict(shard_device=shard_device)
    plans = [ChunkPlan([n], to_divide(s, group_size), dtype, dict(kwargs, rcache_fused=True))
             for n, s in named_sizes if n in private]
    public = [(n, s) for n, s in named_sizes if n not in private]
    groups, block = simple_groups([s for _, s in public], split_number)
    block = to_divide(block, group_size)
    plans += [ChunkPlan([public[i][0] for i in g], block, dtype, dict(kwargs)) for g in groups]
    return SearchResult(ChunkGroup(None), plans)


def get_param_optim_data(param_data: torch.Tensor, param_dtype: torch.dtype, device: torch.device):
    """module.py:21-25: the master copy is fp32, the parameter takes the training dtype."""
    param_data = param_data.to(device)
    optim_data = param_data.clone() if param_data.dtype == torch.float else param_data.float()
    param_data = param_data.to(param_dtype)
    return param_data, optim_data


def reserve_device_pool(nbytes: int, device: torch.device, minimum: int = 1 << 30) -> bool:
    """Takes ``nbytes`` of device memory from the driver in ONE allocation and hands it straight to
    torch's caching allocator, which then carves the chunk shards, master weights and moments out of
    it.  Dozens of allocations of a gigabyte each, made in turn on a device whose memory other
    processes have used and released before, get less contiguous memory than one allocation for all
    of them, and the streaming kernels feel it: the same update launch over the LLaMA-7B set takes
    28.6 ms instead of 29.0-29.3 ms on such a device (28.4 ms either way on a fresh one).  Skipped
    for small sets and when that much memory is not free.  Returns whether it reserved."""
    if nbytes < minimum or device.type != 'cuda':
        return False
    nbytes += 256 << 20    # rounding of the individual allocations, tables, workspaces
    free, _ = torch.cuda.mem_get_info(device)
    cached_free = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
    if nbytes > free + cached_free - (2 << 30):
        return False
    block = torch.empty(nbytes, dtype=torch.uint8, device=device)
    del block    # stays with the caching allocator as one block
    return True


class _Fetcher:
    """The one method of the chunk fetcher the optimizer wrapper calls (fetcher.py)."""

    def __init__(self, group: ChunkGroup):
        self.group = group

    def get_one_chunk(self, tensor: torch.Tensor) -> Chunk:
        return self.group.ten_to_chunk.get(tensor)


class ElixirModule(nn.Module):
    """Chunked storage for the parameters of ``module``.

    args:
        module: the training module, or an ordered mapping ``name -> shape`` for a synthetic
            parameter set whose values are produced in place, directly in the chunk buffers
        search_result: chunk plans (``greedy_search`` builds one)
        dtype: the training dtype: float32, float16, or bfloat16
    """

    def __init__(self,
                 module,
                 search_result: SearchResult,
                 process_group=None,
                 prefetch: bool = False,
                 dtype: torch.dtype = torch.float,
                 reduce_always_fp32: bool = False,
                 output_fp32: bool = False,
                 use_fused_kernels: bool = False,
                 reserve_memory: bool = True) -> None:
        super().__init__()
        assert dtype in {torch.float, torch.float16, torch.bfloat16}
        # Both are speed settings of the reference's forward/backward pass (module.py:51-75: overlapped chunk
        # prefetch, fused LayerNorm / attention); neither changes a result.  That pass is not part of this
        # build, so they are accepted -- the reference's own callers pass them (example/common/elx.py:37)
        # -- and have no effect here.
        self.prefetch_flag = bool(prefetch)
        self.use_fused_kernels = bool(use_fused_kernels)

        self.synthetic = not isinstance(module, nn.Module)
        self.module = module if not self.synthetic else None
        self.dtype = dtype
        self.use_amp = (dtype == torch.float16)
        self.process_group = process_group
        self.reduce_always_fp32 = reduce_always_fp32
        self.output_fp32 = output_fp32
        self.reserve_memory = reserve_memory
        self.buffer = None

        self.no_grad_state_dict = dict()
        self.grad_state_dict: Dict[str, nn.Parameter] = OrderedDict()
        self.param_to_optim: Dict[nn.Parameter, torch.Tensor] = dict()
        self.__init_chunk_group(search_result, module)
        self.fetcher = _Fetcher(self.param_chunk_group)
        # landing during backward: chunks whose gradients are complete land from a hook
        self._landing_in_backward = False
        self._ready: Dict[Chunk, set] = {}
        self._landed: set = set()
        # set by the optimizer step: the shards hold new values that the module's parameters (private
        # copies, as the blocks of the replicated cache are in the reference) have not seen yet
        self._params_stale = False
        if not self.synthetic:
            hooked = set()
            for param in self.grad_state_dict.values():
                if param not in hooked:    # a tied weight is listed under each of its names: one hook all the same
                    hooked.add(param)
                    param.register_post_accumulate_grad_hook(self._gradient_handler)

    def __init_chunk_group(self, sr: SearchResult, module):
        device = gpu_device() if torch.cuda.is_available() else torch.device('cpu')
        if self.synthetic:
            for name, shape in module.items():
                self.grad_state_dict[name] = nn.Parameter(torch.empty(tuple(shape), dtype=self.dtype, device='meta'))
        else:
            state_dict = module.state_dict(keep_vars=True)
            for name, tensor in state_dict.items():
                if isinstance(tensor, nn.Parameter):
                    assert tensor.is_floating_point(), 'the dtypes of parameters should be float dtypes'
                    if tensor.requires_grad:
                        self.grad_state_dict[name] = tensor
                    else:
                        self.no_grad_state_dict[name] = tensor
                        tensor.data = tensor.data.to(dtype=self.dtype, device=device)
                else:
                    to_dtype = self.dtype if tensor.is_floating_point() else tensor.dtype
                    tensor.data = tensor.data.to(dtype=to_dtype, device=device)

        self.param_chunk_group = sr.chunk_group
        self.optim_chunk_group = ChunkGroup(None)
        vis_set = set()
        if self.reserve_memory and device.type == 'cuda':
            gpu_elems = sum(plan.chunk_size for plan in sr.param_chunk_plans
                            if torch.device(plan.kwargs.get('shard_device', device)).type == 'cuda')
            esize = torch.empty(0, dtype=self.dtype).element_size()
            reserve_device_pool(gpu_elems * (esize + 4 + 8), device)    # shards, master, exp_avg, exp_avg_sq

        for plan in sr.param_chunk_plans:
            assert plan.chunk_dtype == self.dtype
            # optimizer chunks should not be gathered
            optim_kwargs = dict(plan.kwargs)
            if 'rcache_fused' in optim_kwargs:
                optim_kwargs['rcache_fused'] = False

            p_chunk = self.param_chunk_group.open_chunk(chunk_size=plan.chunk_size, chunk_dtype=plan.chunk_dtype,
                                                        process_group=self.process_group, chunk_config=plan.kwargs)
            o_chunk = self.optim_chunk_group.open_chunk(chunk_size=plan.chunk_size, chunk_dtype=torch.float,
                                                        process_group=self.process_group, chunk_config=optim_kwargs)

            for name in plan.name_list:
                param = self.grad_state_dict[name]
                if self.synthetic:
                    optim_data = torch.empty(param.shape, dtype=torch.float, device='meta')
                else:
                    param_data, optim_data = get_param_optim_data(param.data, self.dtype, device)
                    param.data = param_data
                p_chunk.append_tensor(param)
                o_chunk.append_tensor(optim_data)
                self.param_to_optim[param] = optim_data
                vis_set.add(param)

            self.param_chunk_group.close_chunk(p_chunk)
            self.optim_chunk_group.close_chunk(o_chunk)
            p_chunk.init_pair(o_chunk)

        # sanity check: every parameter needed gradient has been initialized
        for param in self.grad_state_dict.values():
            assert param in vis_set

        if not self.synthetic:
            self.materialize_params()

    # ------------------------------------------------------------------ parameters and gradients

    def parameters(self, recurse: bool = True):
        if self.synthetic:
            return iter(self.grad_state_dict.values())
        return super().parameters(recurse)

    def named_parameters(self, *args, **kwargs):
        if self.synthetic:
            return iter(self.grad_state_dict.items())
        return super().named_parameters(*args, **kwargs)

    @property
    def param_chunks(self) -> List[Chunk]:
        return self.param_chunk_group.all_chunks

    def materialize_params(self) -> None:
        """Give every parameter of the wrapped module a private copy of its low-precision values
        (what a gather into the replicated cache would expose to the forward pass)."""
        assert not self.synthetic
        self._params_stale = False
        blocks = {}
        for chunk in self.param_chunks:
            if not chunk.optim_sync_flag and torch.cuda.is_available():
                # a host-resident shard whose refresh was deferred: gather source copy with the cast
                # fused in, then the release brings the shard back in sync (chunk.py:264-281)
                block = torch.empty(chunk.chunk_size, dtype=chunk.chunk_dtype, device=gpu_device())
                chunk.replicate(block)
                chunk.scatter(block)
                blocks[chunk] = block
        for param in self.grad_state_dict.values():
            chunk = self.param_chunk_group.ten_to_chunk[param]
            info = chunk.tensors_info[param]
            src = blocks.get(chunk, chunk.shard)
            param.data = src[info.offset:info.end].clone().view(info.fake_data.shape)

    def mark_params_stale(self) -> None:
        """Called by the optimizer step: the next forward pass re-reads the parameters from the shards
        (the reference's forward gathers its chunks anew after every step)."""
        self._params_stale = True

    def forward(self, *args, **kwargs):
        assert not self.synthetic
        if self._params_stale:
            self.materialize_params()
        outputs = self.module(*args, **kwargs)
        if self.output_fp32:
            outputs = outputs.float()
        return outputs

    def _gradient_handler(self, param: nn.Parameter) -> None:
        """module.py:177-190 as a post-accumulate hook: when the last gradient of a chunk has been
        produced, the chunk lands at once (one launch, flags included) and its gradients are freed,
        so that at most one chunk's worth of gradients outlives its producer, as in the reference,
        where a chunk is reduced as soon as all its tensors are ready."""
        if not self._landing_in_backward:
            return
        chunk = self.param_chunk_group.ten_to_chunk[param]
        if chunk.shard_device.type != 'cuda':
            return    # host-resident: lands after backward, through a payload and a transfer
        ready = self._ready.setdefault(chunk, set())
        ready.add(param)
        if len(ready) == chunk.num_tensors:
            land_tensors([chunk], lambda t: t.grad.data.contiguous())
            for t in chunk.tensors_info:
                t.grad = None
            self._landed.add(chunk)
            ready.clear()

    def backward(self, loss: torch.Tensor):
        """module.py:249-254: backward, during which every chunk lands as soon as its gradients are complete."""
        self._backward(loss.backward)

    def backward_by_grad(self, tensor: torch.Tensor, grad: torch.Tensor):
        """Backward from an intermediate tensor and the gradient that arrived for it (what
        ``ElixirOptimizer.backward_by_grad`` calls, optimizer.py:230-236: every stage of a pipeline but the
        last); the chunks land as in ``backward``."""
        self._backward(lambda: torch.autograd.backward(tensor, grad))

    def _backward(self, run) -> None:
        self._landed.clear()
        self._ready.clear()
        self._landing_in_backward = True
        try:
            run()
        finally:
            self._landing_in_backward = False
        self.land_gradients(skip=self._landed)
        self._landed = set()
        self.module.zero_grad(set_to_none=True)

    def land_gradients(self, sync: bool = False, skip=()) -> None:
        """module.py:177-190 + chunk.py:358-393 for one process: every parameter's gradient goes
        into its slice of the chunk's shard, what no parameter covers becomes zero (as the
        replicated block of the reference is after a gather of zero padding), and the flags of every
        chunk are taken in the same pass.  GPU-resident chunks land in one launch straight from the
        ``.grad`` tensors; host-resident ones through a full-size payload and a transfer.  With
        ``sync`` the flags are fetched here, otherwise when somebody reads them (the optimizer step
        does, for all chunks at once)."""
        assert not self.synthetic
        on_gpu = [c for c in self.param_chunks if c.shard_device.type == 'cuda' and c not in skip]
        if on_gpu:

            def grad_of(param):
                assert param.grad is not None, 'every parameter of a chunk needs a gradient before the reduction'
                return param.grad.data.contiguous()

            land_tensors(on_gpu, grad_of)
            if sync:
                for chunk in on_gpu:
                    chunk.update_extra_reduce_info()
        for chunk in self.param_chunks:
            if chunk.shard_device.type == 'cuda' or chunk in skip:
                continue
            payload = torch.zeros(chunk.chunk_size, dtype=chunk.chunk_dtype, device=chunk.shard_device)
            for param, info in chunk.tensors_info.items():
                assert param.grad is not None, 'every parameter of a chunk needs a gradient before the reduction'
                payload[info.offset:info.end].copy_(param.grad.data.flatten())
            chunk.reduce_chunk(payload, always_fp32=self.reduce_always_fp32, sync=sync)

    # ------------------------------------------------------------------ checkpoint of the weights

    def state_dict(self, destination=None, prefix='', keep_vars=False, only_rank_0: bool = False,
                   from_param: bool = False):
        """module.py:258-292: weights come from the fp32 optimizer chunks (or, with ``from_param``,
        from the low-precision chunks), as CPU tensors."""
        assert keep_vars is False, 'state_dict can not keep variables in ElixirModule'
        assert not self.synthetic
        module_state_dict = self.module.state_dict(destination=destination, prefix=prefix, keep_vars=True)
        for name, tensor in module_state_dict.items():
            key = name[len(prefix):]
            if key in self.grad_state_dict:
                param = self.grad_state_dict[key]
                p_chunk = self.param_chunk_group.ten_to_chunk[param]
                info = p_chunk.tensors_info[param]
                src = p_chunk if from_param else p_chunk.paired_chunk
                module_state_dict[name] = src.shard[info.offset:info.end].view(info.fake_data.shape).cpu()
            else:
                module_state_dict[name] = tensor.detach()
        return module_state_dict

    def load_state_dict(self, state_dict: Mapping[str, Any], only_rank_0: bool = False):
        """module.py:294-344: values are written into the fp32 optimizer chunks, then the paired
        low-precision chunks are refreshed."""
        assert not self.synthetic
        touched = set()
        for name, maybe_tensor in state_dict.items():
            if name in self.no_grad_state_dict:
                self.no_grad_state_dict[name].copy_(maybe_tensor)
            elif name in self.grad_state_dict:
                param = self.grad_state_dict[name]
                p_chunk = self.param_chunk_group.ten_to_chunk[param]
                info = p_chunk.tensors_info[param]
                o_chunk = p_chunk.paired_chunk
                o_chunk.shard[info.offset:info.end].copy_(maybe_tensor.data.flatten())
                touched.add(p_chunk)
        for p_chunk in touched:
            p_chunk.optim_update()
        self.materialize_params()
