"""Synthetic chunk sets for measuring the optimizer step: the tensor lists of the model families
packed into chunks with the greedy rule, filled in place on the GPU from a seeded device generator.

Each workload fixes the tensor list, chunk size, low-precision dtype, loss scale, optimizer
settings and the distributions of gradients / master weights / moments.
"""
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import numpy as np
import torch

from . import shapes as S
from .chunk import land_chunks
from .hybrid_adam import HybridAdam
from .module import ElixirModule, greedy_search, reserve_device_pool
from .optimizer import ElixirOptimizer


@dataclass
class WorkloadSpec:
    name: str
    shapes: Callable[[], List[S.NamedShape]]
    chunk_size: int
    dtype: torch.dtype
    loss_scale: float
    grad_std: float          # of the unscaled gradient
    weight_decay: float
    max_norm: float
    lr: float = 1e-3
    betas: Tuple[float, float] = (0.9, 0.999)
    eps: float = 1e-8
    adamw_mode: bool = True
    hysteresis: int = 1
    description: str = ''


WORKLOADS: Dict[str, WorkloadSpec] = {
    # GPT-2 small, fp16, loss scale 64, plain Adam, no clipping
    'c2': WorkloadSpec('c2', S.gpt2_shapes, 64 << 20, torch.float16, 64.0, 1e-3, 0.0, 0.0,
                       description='GPT-2-small 124M, 148 tensors, 2 chunks of 64Mi, fp16 grads x64, Adam wd=0'),
    # OPT-1.3B, bf16, AdamW 0.01 with exempt 1-D tensors, clip 1.0
    'c4': WorkloadSpec('c4', S.opt_shapes, 128 << 20, torch.bfloat16, 1.0, 5e-4, 0.01, 1.0,
                       description='OPT-1.3B, 388 tensors, 11 chunks of 128Mi, bf16 grads, AdamW wd=0.01, clip 1.0'),
    # LLaMA-7B, fp16, dynamic loss scale 2^16, AdamW 0.1, clip 1.0
    'c5': WorkloadSpec('c5', S.llama_shapes, 256 << 20, torch.float16, 65536.0, 1e-3, 0.1, 1.0,
                       description='LLaMA-7B 6.74B, 291 tensors, 27 chunks of 256Mi, fp16 grads x2^16, '
                       'AdamW wd=0.1, clip 1.0'),
}


@dataclass
class BuiltWorkload:
    spec: WorkloadSpec
    module: ElixirModule
    optimizer: ElixirOptimizer
    grads: List[torch.Tensor] = field(default_factory=list)    # one saved gradient buffer per param chunk
    n_valid: int = 0
    n_alloc: int = 0

    def land_gradients(self, fused: bool = False) -> None:
        """Puts the saved gradients back into the low-precision shards (what backward and the
        chunk reduction leave behind) and declares them scaled.  ``fused``: through the landing
        launch that also leaves the flags of every chunk on the device, so that the step needs no
        pass of its own over the gradients; otherwise a plain copy, flags unknown."""
        if fused:
            land_chunks(self.module.param_chunks, self.grads)
        else:
            for pc, g in zip(self.module.param_chunks, self.grads):
                pc.shard.copy_(g)
                pc.invalidate_stats()
        self.optimizer.mark_gradients_scaled()


def build(name: str, device: Optional[torch.device] = None, seed: int = 1234, shapes: Optional[List[S.NamedShape]] = None,
          chunk_size: Optional[int] = None, hysteresis: Optional[int] = None, reserve_memory: bool = True) -> BuiltWorkload:
    spec = WORKLOADS[name]
    device = device or torch.device('cuda', torch.cuda.current_device())
    named = list(shapes if shapes is not None else spec.shapes())
    csize = chunk_size or spec.chunk_size
    sr = greedy_search([(n, S.numel(s)) for n, s in named], csize, spec.dtype, shard_device=device)
    if reserve_memory:
        # everything this workload keeps on the device, the saved gradients included, in one allocation
        esize = torch.empty(0, dtype=spec.dtype).element_size()
        reserve_device_pool(sum(p.chunk_size for p in sr.param_chunk_plans) * (2 * esize + 12), device)
    module = ElixirModule(dict(named), sr, dtype=spec.dtype, reserve_memory=reserve_memory)

    decay, exempt = [], []
    for (pname, shape), p in zip(named, module.parameters()):
        (exempt if S.no_decay(pname, shape) else decay).append(p)
    groups = [dict(params=decay, weight_decay=spec.weight_decay)]
    if exempt:
        groups.append(dict(params=exempt, weight_decay=0.0))
    inner = HybridAdam(groups, lr=spec.lr, betas=spec.betas, eps=spec.eps, weight_decay=spec.weight_decay,
                       adamw_mode=spec.adamw_mode)
    opt = ElixirOptimizer(module, inner, initial_scale=spec.loss_scale,
                          hysteresis=spec.hysteresis if hysteresis is None else hysteresis, max_norm=spec.max_norm)
    if module.use_amp:
        assert opt.loss_scale == spec.loss_scale

    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    built = BuiltWorkload(spec, module, opt)
    piece = 32 << 20    # fill in pieces so that temporaries stay small next to 100+ GB of state
    for pc in module.param_chunks:
        oc = pc.paired_chunk
        used = pc.utilized_size
        m, v = opt._binding.moments(oc)
        g = torch.zeros(pc.shard_size, dtype=spec.dtype, device=device)
        oc.shard.zero_()
        for b in range(0, used, piece):
            e = min(used, b + piece)
            oc.shard[b:e].normal_(0.0, 0.02, generator=gen)
            m[b:e].normal_(0.0, 1e-4, generator=gen)
            v[b:e].uniform_(0.0, 1e-6, generator=gen)
            tmp = torch.empty(e - b, dtype=torch.float32, device=device)
            tmp.normal_(0.0, spec.grad_std * spec.loss_scale, generator=gen)
            g[b:e].copy_(tmp)
            del tmp
        pc.optim_update()
        built.grads.append(g)
        built.n_valid += used
        built.n_alloc += pc.shard_size
    torch.cuda.synchronize(device)
    return built
