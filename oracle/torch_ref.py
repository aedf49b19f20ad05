"""The optimizer step as plain PyTorch CPU ops -- TEST INFRASTRUCTURE ONLY (checker and timed CPU
baseline; never imported by the shipped package).

This is the CPU path the parity target names: ``torch.optim.Adam`` / ``AdamW`` on fp32 tensors,
surrounded by the other stages of ``ElixirOptimizer.step`` as torch ops
(``elixir/wrapper/optimizer.py:137-220``, ``elixir/chunk/core/chunk.py:214-221,403-414``):

    found_inf = isinf(g).any() | isnan(g).any()            on the low-precision gradients
    l2_norm   = g.float().norm(2).item() ** 2               when clipping
    g32       = g.float().div_(combined_scale)              unscale (and clip)
    AdamW / Adam step on (master, exp_avg, exp_avg_sq)
    lowp      = master.to(float16 | bfloat16)               writeback
"""
import math
from typing import Optional

import torch


class TorchCpuStep:

    def __init__(self, master: torch.Tensor, lowp_dtype: torch.dtype, *, lr=1e-3, betas=(0.9, 0.999), eps=1e-8,
                 weight_decay=0.0, adamw_mode=True, exp_avg: Optional[torch.Tensor] = None,
                 exp_avg_sq: Optional[torch.Tensor] = None):
        assert master.device.type == 'cpu' and master.dtype == torch.float32
        self.param = torch.nn.Parameter(master.clone())
        self.lowp_dtype = lowp_dtype
        cls = torch.optim.AdamW if adamw_mode else torch.optim.Adam
        self.optim = cls([self.param], lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, foreach=False)
        if exp_avg is not None:
            st = self.optim.state[self.param]
            st['step'] = torch.tensor(0.0)
            st['exp_avg'] = exp_avg.clone()
            st['exp_avg_sq'] = exp_avg_sq.clone()

    def step(self, grad_lowp: torch.Tensor, loss_scale: float = 1.0, max_norm: float = 0.0):
        """One step on one flat buffer.  Returns (found_inf, lowp copy of the master)."""
        found_inf = bool(torch.isinf(grad_lowp).any().item() | torch.isnan(grad_lowp).any().item())
        if not found_inf:
            combined = loss_scale
            if max_norm > 0.0:
                l2 = grad_lowp.float().norm(2).item()**2
                total_norm = math.sqrt(l2)
                clip = ((total_norm / loss_scale) + 1e-6) / max_norm
                if clip > 1:
                    combined = clip * loss_scale
            g32 = grad_lowp.float()
            if combined != 1:
                g32.div_(combined)
            self.param.grad = g32
            self.optim.step()
            self.param.grad = None
        lowp = self.param.data.to(self.lowp_dtype)
        return found_inf, lowp

    @property
    def master(self) -> torch.Tensor:
        return self.param.data

    @property
    def exp_avg(self) -> torch.Tensor:
        return self.optim.state[self.param]['exp_avg']

    @property
    def exp_avg_sq(self) -> torch.Tensor:
        return self.optim.state[self.param]['exp_avg_sq']
