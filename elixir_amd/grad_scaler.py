"""Loss scalers with the interface the reference's optimizer wrapper drives
(``elixir/wrapper/optimizer.py:76-86,187,197,208``): ``.scale`` (a 1-element fp32 tensor),
``.inv_scale``, ``.update(overflow)``, ``state_dict`` / ``load_state_dict``.

The scale is kept as a host fp32 scalar: reading it never waits for the GPU (the reference holds
it in a device tensor and pays a ``.item()`` per step).  Products are rounded to fp32, so the
trajectory is the one an fp32 tensor would follow.
"""
from typing import Dict, Optional

import numpy as np
import torch


class BaseGradScaler:

    def __init__(self, initial_scale: float, verbose: bool = False):
        assert initial_scale > 0
        self._scale = np.float32(initial_scale)
        self._verbose = verbose

    @property
    def scale(self) -> torch.Tensor:
        return torch.tensor([self._scale], dtype=torch.float32)

    @property
    def scale_value(self) -> float:
        """The scale as a Python float, without building a tensor."""
        return float(self._scale)

    @property
    def inv_scale(self) -> torch.Tensor:
        return self.scale.double().reciprocal().float()

    def state_dict(self) -> Dict:
        return dict(scale=self.scale)

    def load_state_dict(self, state_dict: Dict) -> None:
        self._scale = np.float32(float(state_dict['scale']))

    def update(self, overflow: bool) -> None:
        raise NotImplementedError


class ConstantGradScaler(BaseGradScaler):
    """The scale never changes (optimizer.py:86 uses it with scale 1 for fp32 training)."""

    def __init__(self, initial_scale: float = 1.0, verbose: bool = False):
        super().__init__(initial_scale, verbose)

    def update(self, overflow: bool) -> None:
        pass


class DynamicGradScaler(BaseGradScaler):
    """Dynamic loss scale with hysteresis, as constructed at optimizer.py:78-84.

    On an overflow the hysteresis counter advances and the growth counter resets; once the
    hysteresis counter reaches ``hysteresis`` every further overflow multiplies the scale by
    ``backoff_factor`` (clamped below by ``min_scale``).  After ``growth_interval`` clean steps in
    a row the scale is multiplied by ``growth_factor`` (clamped above by ``max_scale``) and both
    counters reset.
    """

    def __init__(self,
                 initial_scale: float = 2**16,
                 growth_factor: float = 2,
                 backoff_factor: float = 0.5,
                 growth_interval: int = 1000,
                 min_scale: Optional[float] = None,
                 max_scale: Optional[float] = None,
                 hysteresis: int = 2,
                 verbose: bool = False):
        super().__init__(initial_scale, verbose)
        self._min_scale = np.float32(min_scale) if min_scale else None
        self._max_scale = np.float32(max_scale) if max_scale else None
        self._growth_factor = growth_factor
        self._backoff_factor = backoff_factor
        self._growth_interval = growth_interval
        self._growth_step = 0
        self._hysteresis = hysteresis
        self._hysteresis_step = 0
        self._sanity_checks()

    def _sanity_checks(self) -> None:
        if self._min_scale is not None:
            assert self._min_scale > 0, 'The minimum gradient scale cannot be zero or negative'
            assert self._min_scale <= self._scale, 'The minimum gradient scale cannot be greater than the current scale'
        if self._max_scale is not None:
            assert self._max_scale > 0, 'The maximum gradient scale cannot be zero or negative'
            assert self._max_scale >= self._scale, 'The maximum gradient scale cannot be smaller than the current scale'
        assert self._growth_factor > 1, 'The growth factor cannot be equal or smaller than 1'
        assert 0 < self._backoff_factor < 1, 'The backoff factor must be between 0 and 1'
        assert self._hysteresis >= 0, 'The hysteresis cannot be negative'

    def update(self, overflow: bool) -> None:
        if overflow:
            self._hysteresis_step += 1
            self._growth_step = 0
            if self._hysteresis_step >= self._hysteresis:
                self._backoff_scale()
        else:
            self._growth_step += 1
            if self._growth_step == self._growth_interval:
                self._growth_step = 0
                self._hysteresis_step = 0
                self._grow_scale()

    def _backoff_scale(self) -> None:
        self._scale = np.float32(self._scale * np.float32(self._backoff_factor))
        if self._min_scale is not None:
            self._scale = max(self._scale, self._min_scale)

    def _grow_scale(self) -> None:
        self._scale = np.float32(self._scale * np.float32(self._growth_factor))
        if self._max_scale is not None:
            self._scale = min(self._scale, self._max_scale)

    def state_dict(self) -> Dict:
        """The scale, the factors and the hysteresis as the scaler this class mirrors saves them, and
        what a resumed run needs besides: both counters, the growth interval and the clamps."""
        return dict(scale=self.scale, growth_factor=self._growth_factor, backoff_factor=self._backoff_factor,
                    hysteresis=self._hysteresis, growth_step=self._growth_step,
                    hysteresis_step=self._hysteresis_step, growth_interval=self._growth_interval,
                    min_scale=None if self._min_scale is None else float(self._min_scale),
                    max_scale=None if self._max_scale is None else float(self._max_scale))

    def load_state_dict(self, state_dict: Dict) -> None:
        self._scale = np.float32(float(state_dict['scale']))
        self._growth_factor = state_dict['growth_factor']
        self._backoff_factor = state_dict['backoff_factor']
        self._hysteresis = state_dict['hysteresis']
        self._growth_step = state_dict.get('growth_step', 0)
        self._hysteresis_step = state_dict.get('hysteresis_step', 0)
        self._growth_interval = state_dict.get('growth_interval', self._growth_interval)
        if 'min_scale' in state_dict:
            self._min_scale = None if state_dict['min_scale'] is None else np.float32(state_dict['min_scale'])
        if 'max_scale' in state_dict:
            self._max_scale = None if state_dict['max_scale'] is None else np.float32(state_dict['max_scale'])
