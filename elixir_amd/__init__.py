"""MI355X-native implementation of Elixir's optimizer step over chunk-packed parameters.

The public names mirror the reference's for this path: ``ElixirModule`` (chunk pairing only),
``ElixirOptimizer``, ``HybridAdam``, ``Chunk`` / ``ChunkGroup``, the loss scalers, and the chunk
plan types.  The device work runs in ``libelx_hip.so`` (hand-written HIP for gfx950) through the C
ABI declared in ``include/elx_abi.h``; there is no CPU or eager-PyTorch fallback.
"""
from .chunk import Chunk, ChunkFullError, ChunkGroup, TensorInfo, TensorState
from .grad_scaler import BaseGradScaler, ConstantGradScaler, DynamicGradScaler
from .hybrid_adam import CPUAdam, FusedAdam, HybridAdam
from .module import (ChunkPlan, ElixirModule, SearchResult, greedy_groups, greedy_search, simple_groups,
                     simple_search)
from .optimizer import ElixirOptimizer, OptimState, calc_combined_scale

__all__ = [
    'Chunk', 'ChunkFullError', 'ChunkGroup', 'TensorInfo', 'TensorState', 'BaseGradScaler', 'ConstantGradScaler',
    'DynamicGradScaler', 'HybridAdam', 'FusedAdam', 'CPUAdam', 'ChunkPlan', 'ElixirModule', 'SearchResult', 'greedy_groups', 'greedy_search',
    'simple_groups', 'simple_search', 'ElixirOptimizer', 'OptimState', 'calc_combined_scale'
]
