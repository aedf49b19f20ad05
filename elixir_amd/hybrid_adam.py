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
there is no CPU path.
"""
import math
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from . import _abi
from .chunk import Chunk, DeviceTable, dtype_code


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


class _CachedTable:
    """Device copy of a host table, re-uploaded only when the host contents change."""

    def __init__(self):
        self.table: Optional[DeviceTable] = None

    def get(self, host: np.ndarray, device: torch.device) -> DeviceTable:
        t = self.table
        if t is None or t.dev.device != device or t.host.shape != host.shape or t.host.tobytes() != host.tobytes():
            self.table = DeviceTable(host.copy(), device)
        return self.table


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
        for c in self.chunks:
            if c.shard_device.type != 'cuda':
                raise RuntimeError('HybridAdam runs on the GPU: optimizer shards must live in device memory '
                                   '(host-resident shards are not supported by this build)')

    def moments(self, chunk: Chunk) -> Tuple[torch.Tensor, torch.Tensor]:
        if chunk not in self.flat_m:
            self.flat_m[chunk] = torch.zeros(chunk.shard_size, dtype=torch.float32, device=chunk.shard_device)
            self.flat_v[chunk] = torch.zeros(chunk.shard_size, dtype=torch.float32, device=chunk.shard_device)
        return self.flat_m[chunk], self.flat_v[chunk]


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
        self._chunk_table = _CachedTable()
        self._seg_table = _CachedTable()
        self._hyper_table = _CachedTable()
        self._checked_key = None
        self._checked = None

    # ------------------------------------------------------------------ chunk binding

    def bind_chunks(self, ranges: Dict[torch.nn.Parameter, Tuple[Chunk, int, int]]) -> ChunkBinding:
        """Called by ``ElixirOptimizer``: ``ranges[fake_param] = (optim_chunk, begin, end)``."""
        self._binding = ChunkBinding(ranges)
        return self._binding

    @property
    def binding(self) -> Optional[ChunkBinding]:
        return self._binding

    # ------------------------------------------------------------------ the step

    def _hyper_index(self, hypers: Dict, group: Dict, step: int) -> int:
        beta1, beta2 = group['betas']
        key = (group['lr'], beta1, beta2, group['eps'], group['weight_decay'], step, group['bias_correction'])
        idx = hypers.get(key)
        if idx is None:
            idx = len(hypers)
            hypers[key] = idx
        return idx

    @torch.no_grad()
    def step(self, closure=None, div_scale: float = -1):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        hypers: Dict = {}
        if self._binding is not None:
            launch = self._collect_bound(hypers)
        else:
            launch = self._collect_standalone(hypers)
        if launch is None:
            return loss
        chunks, segs, grad_code, lowp_code, device = launch

        hyper_host = np.concatenate([
            make_hyper_record(lr, b1, b2, eps, wd, step, bc, self.adamw_mode)
            for (lr, b1, b2, eps, wd, step, bc) in hypers.keys()
        ])

        key = (chunks.tobytes(), segs.tobytes(), len(hyper_host), grad_code, lowp_code)
        if key != self._checked_key:
            self._checked = _abi.check_tables(chunks, segs, len(hyper_host), grad_code, lowp_code)
            self._checked_key = key
        info = self._checked

        d_chunks = self._chunk_table.get(chunks, device)
        d_segs = self._seg_table.get(segs, device)
        d_hypers = self._hyper_table.get(hyper_host, device)
        stream = torch.cuda.current_stream(device).cuda_stream
        _abi.adam_step_mt(d_chunks.ptr, len(chunks), d_segs.ptr, len(segs), d_hypers.ptr, len(hyper_host), info,
                          float(div_scale), grad_code, lowp_code, self.blocks_per_cu, stream)
        if self._binding is not None and lowp_code != _abi.ELX_NONE:
            self._binding.fused_writeback = True
        return loss

    def _collect_bound(self, hypers: Dict):
        b = self._binding
        b.require_gpu()
        n_chunks = len(b.chunks)
        chunks = np.zeros(n_chunks, dtype=_abi.CHUNK_DTYPE)
        per_chunk: List[List[Tuple[int, int, int]]] = [[] for _ in range(n_chunks)]
        for group in self.param_groups:
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
                state['step'] += 1
                per_chunk[b.chunk_index[chunk]].append((begin, end, self._hyper_index(hypers, group, state['step'])))

        n_segs = sum(len(x) for x in per_chunk)
        if n_segs == 0:
            return None
        segs = np.zeros(n_segs, dtype=_abi.SEG_DTYPE)
        tile = _abi.tile_elems()
        pos, tiles = 0, 0
        lowp_dtype = b.chunks[0].paired_chunk.chunk_dtype
        for i, c in enumerate(b.chunks):
            pc = c.paired_chunk
            assert pc.chunk_dtype == lowp_dtype, 'all parameter chunks of one optimizer share a dtype'
            flat_m, flat_v = b.moments(c)
            row = chunks[i]
            row['grad'] = 0 if b.zero_grads else pc.shard.data_ptr()
            row['lowp_out'] = 0 if b.zero_grads else pc.shard.data_ptr()
            row['master'] = c.shard.data_ptr()
            row['m'] = flat_m.data_ptr()
            row['v'] = flat_v.data_ptr()
            row['n_alloc'] = c.shard_size
            row['n_valid'] = pc.n_valid
            row['tile_begin'] = tiles
            tiles += (c.shard_size + tile - 1) // tile
            row['seg_begin'] = pos
            for begin, end, h in sorted(per_chunk[i]):
                segs[pos] = (begin, end, h, 0)
                pos += 1
            row['seg_end'] = pos
        code = dtype_code(lowp_dtype)
        return chunks, segs, code, (_abi.ELX_NONE if b.zero_grads else code), b.chunks[0].shard_device

    def _collect_standalone(self, hypers: Dict):
        rows = []
        grad_dtype = None
        device = None
        for group in self.param_groups:
            for p in group['params']:
                if p.grad is None:
                    continue
                if p.numel() == 0:
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
                state['step'] += 1
                rows.append((p, state, self._hyper_index(hypers, group, state['step'])))
        if not rows:
            return None
        chunks = np.zeros(len(rows), dtype=_abi.CHUNK_DTYPE)
        segs = np.zeros(len(rows), dtype=_abi.SEG_DTYPE)
        tile = _abi.tile_elems()
        tiles = 0
        for i, (p, state, h) in enumerate(rows):
            n = p.numel()
            row = chunks[i]
            row['grad'] = p.grad.data_ptr()
            row['lowp_out'] = 0
            row['master'] = p.data.data_ptr()
            row['m'] = state['exp_avg'].data_ptr()
            row['v'] = state['exp_avg_sq'].data_ptr()
            row['n_alloc'] = n
            row['n_valid'] = n
            row['tile_begin'] = tiles
            tiles += (n + tile - 1) // tile
            row['seg_begin'] = i
            row['seg_end'] = i + 1
            segs[i] = (0, n, h, 0)
        return chunks, segs, dtype_code(grad_dtype), _abi.ELX_NONE, device
