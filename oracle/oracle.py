"""CPU oracle for the ElixirOptimizer.step path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
The shipped package (elixir_amd/) never imports it and has no CPU fallback.

Two halves:

* thin numpy wrappers over ``elx_oracle.c`` (element-wise arithmetic: overflow flag, squared
  norm, Adam/AdamW with fused unscale, low-precision writeback);
* a pure-Python restatement of the host control flow of the reference's step
  (``elixir/wrapper/optimizer.py:137-220``), of the loss-scale state machine it drives, of the
  chunk layout rules (``elixir/chunk/core/chunk.py:223-262``) and of the greedy packing rule
  (``elixir/search/mini_waste.py:78-96``).

Low-precision arrays are carried as ``numpy.uint16`` bit patterns (numpy has no bfloat16).
dtype codes: 0 = fp32, 1 = fp16, 2 = bf16.
"""
import ctypes
import math
import os
import subprocess
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, '_build', 'libelx_oracle.so')

F32, F16, BF16 = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile elx_oracle.c with the committed Makefile; returns the library path."""
    src = os.path.join(_HERE, 'elx_oracle.c')
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(['make', '-C', _HERE, '-B', '-s'])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u64, i64, dbl, flt, cint = (ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int64, ctypes.c_double,
                                        ctypes.c_float, ctypes.c_int)
        L.orc_lowp_to_f32.restype = flt
        L.orc_lowp_to_f32.argtypes = [ctypes.c_uint16, cint]
        L.orc_f32_to_lowp.restype = ctypes.c_uint16
        L.orc_f32_to_lowp.argtypes = [flt, cint]
        L.orc_lowp_to_f32_array.restype = None
        L.orc_lowp_to_f32_array.argtypes = [vp, vp, cint, u64]
        L.orc_overflow.restype = cint
        L.orc_overflow.argtypes = [vp, cint, u64]
        L.orc_sumsq.restype = dbl
        L.orc_sumsq.argtypes = [vp, cint, u64]
        L.orc_l2norm_sq_ref.restype = dbl
        L.orc_l2norm_sq_ref.argtypes = [vp, cint, u64]
        L.orc_writeback.restype = None
        L.orc_writeback.argtypes = [vp, vp, cint, u64]
        L.orc_land.restype = None
        L.orc_land.argtypes = [vp, cint, vp, cint, u64, flt]
        L.orc_adam.restype = None
        L.orc_adam.argtypes = [vp, cint, vp, vp, vp, u64, dbl, dbl, dbl, dbl, dbl, i64, cint, cint, flt]
        L.orc_adam_f64.restype = None
        L.orc_adam_f64.argtypes = [vp, cint, vp, vp, vp, vp, vp, vp, u64, dbl, dbl, dbl, dbl, dbl, i64, cint, cint, dbl]
        L.orc_num_threads.restype = cint
        _lib = L
    return _lib


def _ptr(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.flags['C_CONTIGUOUS']
    return a.ctypes.data_as(ctypes.c_void_p)


def _check_grad(g: np.ndarray, dtype: int):
    want = np.float32 if dtype == F32 else np.uint16
    assert g.dtype == want, f'grad array must be {want} for dtype code {dtype}'


# ---------------------------------------------------------------------------------------------
# element-wise arithmetic (elx_oracle.c)
# ---------------------------------------------------------------------------------------------


def lowp_to_f32(bits: np.ndarray, dtype: int) -> np.ndarray:
    """Exact upcast of fp16/bf16 bit patterns to fp32."""
    flat = np.ascontiguousarray(bits, dtype=np.uint16).ravel()
    out = np.empty(flat.shape, dtype=np.float32)
    lib().orc_lowp_to_f32_array(_ptr(flat), _ptr(out), dtype, flat.size)
    return out.reshape(np.shape(bits))


def overflow(g: np.ndarray, dtype: int) -> bool:
    """chunk.py:214-216 -- any(isinf) | any(isnan) over the given (valid) elements."""
    _check_grad(g, dtype)
    return bool(lib().orc_overflow(_ptr(g), dtype, g.size))


def sumsq(g: np.ndarray, dtype: int) -> float:
    """float64 sum of squares (brute force)."""
    _check_grad(g, dtype)
    return float(lib().orc_sumsq(_ptr(g), dtype, g.size))


def l2norm_sq_ref(g: np.ndarray, dtype: int) -> float:
    """chunk.py:218-221 -- (fp32 norm).item()**2."""
    _check_grad(g, dtype)
    return float(lib().orc_l2norm_sq_ref(_ptr(g), dtype, g.size))


def writeback(master: np.ndarray, dtype: int) -> np.ndarray:
    """chunk.py:403-414 -- cast an fp32 shard to the low-precision dtype (RNE)."""
    assert master.dtype == np.float32
    out = np.empty(master.shape, dtype=np.float32 if dtype == F32 else np.uint16)
    lib().orc_writeback(_ptr(master), _ptr(out), dtype, master.size)
    return out


def land(src: np.ndarray, src_dtype: int, dst_dtype: int, mul: float = 1.0) -> np.ndarray:
    """chunk.py:299,309-315,484-489 -- the payload as it sits in the shard after landing: scaled by
    ``mul`` in the payload's own type (``mul = float32(1/pg_size)``; 1.0 on one GPU), then cast to
    the shard's type."""
    _check_grad(src, src_dtype)
    assert src_dtype == dst_dtype or src_dtype == F32
    out = np.empty(src.shape, dtype=np.float32 if dst_dtype == F32 else np.uint16)
    lib().orc_land(_ptr(src), src_dtype, _ptr(out), dst_dtype, src.size, float(np.float32(mul)))
    return out


def adam(g: Optional[np.ndarray],
         g_dtype: int,
         p: np.ndarray,
         m: np.ndarray,
         v: np.ndarray,
         *,
         lr: float,
         beta1: float,
         beta2: float,
         eps: float,
         weight_decay: float,
         step: int,
         adamw_mode: bool,
         bias_correction: bool = True,
         div_scale: float = -1.0) -> None:
    """In-place fp32 Adam/AdamW step with fused unscale; see orc_adam."""
    if g is not None:
        _check_grad(g, g_dtype)
        assert g.size == p.size
    for a in (p, m, v):
        assert a.dtype == np.float32 and a.size == p.size
    lib().orc_adam(_ptr(g), g_dtype, _ptr(p), _ptr(m), _ptr(v), p.size, lr, beta1, beta2, eps, weight_decay,
                   int(step), int(adamw_mode), int(bias_correction), float(div_scale))


def adam_f64(g, g_dtype, p, m, v, *, lr, beta1, beta2, eps, weight_decay, step, adamw_mode, bias_correction=True,
             div_scale=-1.0):
    """float64 closed form of the same step; returns (p, m, v) as float64 arrays."""
    if g is not None:
        _check_grad(g, g_dtype)
    po, mo, vo = (np.empty(p.shape, dtype=np.float64) for _ in range(3))
    lib().orc_adam_f64(_ptr(g), g_dtype, _ptr(p), _ptr(m), _ptr(v), _ptr(po), _ptr(mo), _ptr(vo), p.size, lr, beta1,
                       beta2, eps, weight_decay, int(step), int(adamw_mode), int(bias_correction), float(div_scale))
    return po, mo, vo


def num_threads() -> int:
    return int(lib().orc_num_threads())


# ---------------------------------------------------------------------------------------------
# loss-scale state machine
# ---------------------------------------------------------------------------------------------


class DynamicGradScalerOracle:
    """Restatement of the dynamic loss scaler the reference constructs at
    ``elixir/wrapper/optimizer.py:78-84``.  The class itself lives in ColossalAI (not in the
    reference tree); its published rule is:

        update(overflow):
          overflow:  hysteresis_step += 1; growth_step = 0
                     if hysteresis_step >= hysteresis: scale = max(scale*backoff, min_scale)
          otherwise: growth_step += 1
                     if growth_step == growth_interval:
                         growth_step = 0; hysteresis_step = 0
                         scale = min(scale*growth, max_scale)

    The scale is an fp32 scalar, so products are rounded to fp32.
    """

    def __init__(self, initial_scale=2**16, growth_factor=2, backoff_factor=0.5, growth_interval=1000,
                 min_scale=None, max_scale=None, hysteresis=2):
        self.scale = np.float32(initial_scale)
        self.min_scale = None if not min_scale else np.float32(min_scale)
        self.max_scale = None if not max_scale else np.float32(max_scale)
        self.growth_factor = growth_factor
        self.backoff_factor = backoff_factor
        self.growth_interval = growth_interval
        self.hysteresis = hysteresis
        self.growth_step = 0
        self.hysteresis_step = 0

    def update(self, overflow: bool) -> None:
        if overflow:
            self.hysteresis_step += 1
            self.growth_step = 0
            if self.hysteresis_step >= self.hysteresis:
                self.scale = np.float32(self.scale * np.float32(self.backoff_factor))
                if self.min_scale is not None:
                    self.scale = max(self.scale, self.min_scale)
        else:
            self.growth_step += 1
            if self.growth_step == self.growth_interval:
                self.growth_step = 0
                self.hysteresis_step = 0
                self.scale = np.float32(self.scale * np.float32(self.growth_factor))
                if self.max_scale is not None:
                    self.scale = min(self.scale, self.max_scale)


class ConstantGradScalerOracle:
    """``ConstantGradScaler(1.0)`` of optimizer.py:86: the scale never moves."""

    def __init__(self, scale=1.0):
        self.scale = np.float32(scale)

    def update(self, overflow: bool) -> None:
        pass


# ---------------------------------------------------------------------------------------------
# host scalars of the step
# ---------------------------------------------------------------------------------------------


def global_norm(chunk_l2_norms: Sequence[float]) -> float:
    """optimizer.py:149-164 on one process: the per-chunk squared norms are summed in a Python
    float, pass through a 1-element fp32 buffer (``_comm_buffer.fill_`` / ``.item()``) and the
    square root is taken in float64."""
    part = 0.0
    for x in chunk_l2_norms:
        part += x
    norm_sqr = 0.0
    norm_sqr += float(np.float32(part))
    return math.sqrt(norm_sqr)


def combined_scale(loss_scale: float, total_norm: Optional[float], max_norm: float) -> float:
    """optimizer.py:166-183.  ``total_norm`` is None when clipping is off."""
    combined = loss_scale
    if max_norm > 0.0:
        clip = ((total_norm / loss_scale) + 1e-6) / max_norm
        if clip > 1:
            combined = clip * loss_scale
    if combined == 1:
        return -1
    return combined


# ---------------------------------------------------------------------------------------------
# chunk layout
# ---------------------------------------------------------------------------------------------


def greedy_pack(sizes: Sequence[int], chunk_size: int) -> List[List[int]]:
    """mini_waste.py:78-96 -- walk the tensors in order; open a new chunk whenever the space
    left in the current one is smaller than the next tensor.  Returns lists of tensor indices."""
    groups: List[List[int]] = []
    left = 0
    for i, s in enumerate(sizes):
        if left < s:
            left = chunk_size
            groups.append([])
        assert left >= s, 'tensor larger than the chunk'
        left -= s
        groups[-1].append(i)
    return groups


def simple_pack(sizes: Sequence[int], private: Sequence[bool], group_size: int,
                split_number: int) -> Tuple[List[int], List[List[int]], int]:
    """search/simple.py:30-74 with search/base.py:87-108 -- the plan of ``simple_search``: every
    private tensor (one a model uses more than once, search/utils.py:24-33) gets a chunk of its own,
    its size rounded up to a multiple of ``group_size``; the public tensors, in order, are cut into
    ``min(count, split_number)`` runs by count (the remainder goes one each to the first runs) and every
    public chunk has the size of the fullest run, rounded up the same way.

    Returns (private chunk sizes, public groups as index lists into ``sizes``, public chunk size)."""
    def to_divide(a, b):    # search/utils.py:5-6
        return a + (-a % b)

    private_sizes = [to_divide(s, group_size) for s, p in zip(sizes, private) if p]
    public = [i for i, p in enumerate(private) if not p]
    split_number = min(len(public), split_number)
    groups: List[List[int]] = []
    block = 0
    if split_number > 0:
        average, left = divmod(len(public), split_number)
        at = 0
        for i in range(split_number):
            count = average + (1 if i < left else 0)
            groups.append(public[at:at + count])
            at += count
        block = max(sum(sizes[i] for i in g) for g in groups)
    return private_sizes, groups, to_divide(block, group_size)


def chunk_offsets(sizes: Sequence[int]) -> List[Tuple[int, int]]:
    """chunk.py:223-247 -- tensors are appended back to back with no alignment padding."""
    out, used = [], 0
    for s in sizes:
        out.append((used, used + s))
        used += s
    return out


def valid_end(utilized_size: int, shard_begin: int, shard_size: int) -> int:
    """chunk.py:78,249-257 -- number of meaningful elements at the head of the shard; stays at the
    sentinel ``shard_size + 1`` when the shard is completely used (slicing then takes it whole)."""
    shard_end = shard_begin + shard_size
    ve = shard_size + 1
    if utilized_size <= shard_begin:
        ve = 0
    elif utilized_size < shard_end:
        ve = utilized_size - shard_begin
    return ve


def range_pair(offset: int, end: int, shard_begin: int, shard_size: int) -> Tuple[int, int]:
    """optimizer.py:240-244 -- a tensor's slice clipped to this rank's shard."""
    return max(0, offset - shard_begin), min(shard_size, end - shard_begin)


# ---------------------------------------------------------------------------------------------
# the whole step, on numpy arrays
# ---------------------------------------------------------------------------------------------


@dataclass
class OracleSegment:
    """One tensor's slice of a chunk and the hyper-parameters of the group it belongs to."""
    begin: int
    end: int
    lr: float = 1e-3
    betas: Tuple[float, float] = (0.9, 0.999)
    eps: float = 1e-8
    weight_decay: float = 0.0
    bias_correction: bool = True
    step: int = 0    # state['step'] of this tensor: number of non-skipped updates so far


@dataclass
class OracleChunk:
    """A paired (low-precision, fp32) chunk on one process: ``lowp`` plays the param shard that
    holds the gradients at step time, ``master`` the fp32 optimizer shard; m/v are flat."""
    lowp: np.ndarray    # uint16 bits (fp16/bf16) or float32
    master: np.ndarray
    m: np.ndarray
    v: np.ndarray
    valid_end: int
    segments: List[OracleSegment] = field(default_factory=list)


def reference_step(chunks: List[OracleChunk], lowp_dtype: int, scaler, *, max_norm: float = 0.0,
                   adamw_mode: bool = True) -> Dict:
    """Restatement of ``ElixirOptimizer.step`` (optimizer.py:192-220) on one process, with the
    flags of ``Chunk.update_extra_reduce_info`` (chunk.py:345-356) evaluated first.

    Mutates the chunks in place and returns what the step decided."""
    clipping = max_norm > 0.0
    flags, norms = [], []
    for c in chunks:
        valid = c.lowp[:c.valid_end]
        flags.append(overflow(valid, lowp_dtype))
        norms.append(l2norm_sq_ref(valid, lowp_dtype) if clipping else None)

    found_inf = sum(int(f) for f in flags) > 0    # optimizer.py:137-142
    if found_inf:
        scaler.update(True)    # optimizer.py:196-203
        for c in chunks:
            c.lowp[:] = writeback(c.master, lowp_dtype)
        return dict(found_inf=True, combined_scale=None, loss_scale=float(scaler.scale), total_norm=None)

    loss_scale = float(scaler.scale)
    total_norm = global_norm(norms) if clipping else None
    comb = combined_scale(loss_scale, total_norm, max_norm)
    scaler.update(False)    # optimizer.py:208

    for c in chunks:
        for s in c.segments:
            s.step += 1
            sl = slice(s.begin, s.end)
            # the slices are views: the update lands in the chunk arrays
            adam(c.lowp[sl], lowp_dtype, c.master[sl], c.m[sl], c.v[sl], lr=s.lr, beta1=s.betas[0],
                 beta2=s.betas[1], eps=s.eps, weight_decay=s.weight_decay, step=s.step, adamw_mode=adamw_mode,
                 bias_correction=s.bias_correction, div_scale=float(comb))
    for c in chunks:    # optimizer.py:219 -> chunk.py:414, the whole shard incl. padding
        c.lowp[:] = writeback(c.master, lowp_dtype)
    return dict(found_inf=False, combined_scale=comb, loss_scale=float(scaler.scale), total_norm=total_norm)
