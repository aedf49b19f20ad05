"""Host-side planning of the update launch.

The update kernel runs best as a 2-D grid ``(tiles per record, records)`` whose records are
equal-sized blocks: no lookup to find a tile's owner, very few workgroups without work, and a
segment table of one or two entries per record.  Runs of pure padding at the end of a shard are
left out of that launch and refreshed by the wide-workgroup refresh launch instead.

``build_plan`` turns a list of flat buffers (a chunk shard, or a standalone parameter) with their
segments into
  * ``rows`` / ``segs``: the ElxChunk / ElxSeg tables of the update launch, one row per block of
    ``block_elems`` elements that contains at least one valid element;
  * ``refresh_rows``: ElxChunk rows (lowp_out, master, n_alloc only) for the padding runs, cut into
    blocks of the same size, or None.
"""
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _abi

MAX_ROWS = 32768    # target upper bound on update rows (the grid's y extent must stay below 65536)


@dataclass
class FlatBuffer:
    """One flat run of elements: a chunk shard pair or a standalone parameter."""
    grad: int         # device address of the gradients (0: zero gradient)
    lowp_out: int     # device address of the low-precision copy (0: none)
    master: int
    m: int
    v: int
    n_alloc: int
    n_valid: int
    segs: List[Tuple[int, int, int]] = field(default_factory=list)    # (begin, end, hyper), sorted, disjoint


@dataclass
class LaunchPlan:
    rows: np.ndarray
    segs: np.ndarray
    refresh_rows: Optional[np.ndarray]
    refresh_max_elems: int
    block_elems: int
    info: _abi.TableInfo


def _pow2_at_least(x: int) -> int:
    p = 1
    while p < x:
        p <<= 1
    return p


BLOCK_TILES = 2048  # tiles per block the update launch streams best with (measured: the GPT-2, OPT and LLaMA sets agree)


def choose_block_elems(buffers: Sequence[FlatBuffer], tile: int) -> int:
    """A power-of-two multiple of the tile: BLOCK_TILES tiles, more only when the launch would
    otherwise exceed about MAX_ROWS / 2 rows, less (down to 16 tiles) when no buffer is that long."""
    total = sum(min(b.n_alloc, b.n_valid + tile) for b in buffers)
    longest = max((b.n_alloc for b in buffers), default=0)
    block = max(BLOCK_TILES * tile, _pow2_at_least((total + MAX_ROWS // 2 - 1) // (MAX_ROWS // 2)))
    return max(16 * tile, min(block, _pow2_at_least(longest)))


# The update launch writes the low-precision copy with stores that the memory-side cache (256 MiB) takes in
# when all low-precision shards of the launch together are no larger than this many bytes.  Measured on sets
# of equal tensors, step time with against without: -2.5 % at 128 MB, -3 to -5 % at 512 MB, -1.5 % at 1 GB,
# -1.1 % at 2 GB, -0.5 % at 2.9 GB (the same whether the gradients are re-landed between the steps or the
# steps follow each other back to back); on the OPT-1.3B set (2.95 GB) +0.2 %, on LLaMA-7B (14.5 GB) +1 %:
# there the streaming stores are the better ones.
KEEP_LOWP_CACHED_BELOW = 2 << 30

# Everything an update launch touches -- gradients, master weights, exp_avg, exp_avg_sq, low-precision copy --
# is at most this many bytes: the size of the memory-side cache.  The launch then reads with ordinary loads
# and stores everything the way it stores the low-precision copy above, and the next step finds the state in
# the cache.  Measured on a flat fp32 parameter with fp32 gradients, step time with against without: 0.0363 /
# 0.0405 ms at 4 Mi elements, 0.0548 / 0.0544 at 8 Mi, 0.0845 / 0.0906 at 16 Mi (256 MiB in all: the limit);
# beyond it the policy loses: 0.1043 / 0.1044 at 19.9 Mi, 0.1264 / 0.1204 at 23.7 Mi, 0.1805 / 0.1581 at 32 Mi.
KEEP_STATE_CACHED_BELOW = 256 << 20

FOLD_PADDING_BELOW = 24 << 20    # elements: about 20 us of refresh, less than what a launch of its own costs a small set


def build_plan(buffers: Sequence[FlatBuffer], grad_esize: int, lowp_esize: int, n_hypers: int, grad_dtype: int,
               lowp_dtype: int, fold_padding_below: int = FOLD_PADDING_BELOW, device_resident: bool = True) -> LaunchPlan:
    """``fold_padding_below``: when the runs of pure padding hold fewer elements than this in total they
    are listed as rows of the update launch (n_valid = 0: refreshed tile by tile there) instead of going
    to a refresh launch of their own.  ``device_resident``: every buffer lies in device memory (the
    memory-side cache only fronts that)."""
    tile = _abi.tile_elems()
    block = choose_block_elems(buffers, tile)
    rows, segs, refresh = [], [], []
    tiles = 0
    padding = sum(max(0, b.n_alloc - min(b.n_alloc, -(-b.n_valid // block) * block)) for b in buffers if b.lowp_out)
    fold = 0 < padding < fold_padding_below
    for buf in buffers:
        assert 0 <= buf.n_valid <= buf.n_alloc
        # the update covers whole blocks up to the one that holds the last valid element (and, when the
        # padding is folded in, the rest of the buffer as well)
        up_end = min(buf.n_alloc, -(-buf.n_valid // block) * block)
        if fold and buf.lowp_out:
            up_end = buf.n_alloc
        seg_arr = np.array(buf.segs, dtype=np.int64).reshape(-1, 3)
        if len(seg_arr):
            assert np.all(seg_arr[:, 0] < seg_arr[:, 1]) and np.all(seg_arr[1:, 0] >= seg_arr[:-1, 1]), \
                'segments must be sorted, non-empty and disjoint'
            assert seg_arr[-1, 1] <= buf.n_valid, 'a segment reaches beyond the valid head of its buffer'
        for b in range(0, up_end, block):
            n = min(block, up_end - b)
            seg_begin = len(segs)
            if len(seg_arr):
                lo = int(np.searchsorted(seg_arr[:, 1], b, side='right'))       # first segment ending after b
                hi = int(np.searchsorted(seg_arr[:, 0], b + n, side='left'))    # first segment starting at/after the end
                for sb, se, h in seg_arr[lo:hi]:
                    segs.append((max(int(sb), b) - b, min(int(se), b + n) - b, int(h), 0))
            rows.append((buf.grad + b * grad_esize if buf.grad else 0, buf.lowp_out + b * lowp_esize if buf.lowp_out else 0,
                         buf.master + 4 * b, buf.m + 4 * b, buf.v + 4 * b, n, max(0, min(n, buf.n_valid - b)), tiles,
                         seg_begin, len(segs)))
            tiles += (n + tile - 1) // tile
        if buf.lowp_out:
            # the run of pure padding, in blocks of the same size: an even grid for the refresh launch
            for b in range(up_end, buf.n_alloc, block):
                refresh.append((0, buf.lowp_out + b * lowp_esize, buf.master + 4 * b, buf.master + 4 * b,
                                buf.master + 4 * b, min(block, buf.n_alloc - b), 0, 0, 0, 0))
    rows_np = np.array(rows, dtype=_abi.CHUNK_DTYPE) if rows else np.zeros(0, dtype=_abi.CHUNK_DTYPE)
    segs_np = np.array(segs, dtype=_abi.SEG_DTYPE) if segs else np.zeros(0, dtype=_abi.SEG_DTYPE)
    info = _abi.check_tables(rows_np, segs_np, n_hypers, grad_dtype, lowp_dtype) if len(rows_np) else None
    if info is not None:
        lowp_bytes = sum(b.n_alloc for b in buffers if b.lowp_out) * lowp_esize
        state_bytes = sum(b.n_alloc * (12 + (grad_esize if b.grad else 0)
                                       + (lowp_esize if b.lowp_out and b.lowp_out != b.grad else 0)) for b in buffers)
        policy = 0
        if device_resident and 0 < lowp_bytes <= KEEP_LOWP_CACHED_BELOW:
            policy = 1
        if device_resident and state_bytes <= KEEP_STATE_CACHED_BELOW:
            policy = 2
        info = info.with_cache_policy(policy)
    refresh_np, refresh_max = None, 0
    if refresh:
        refresh_np = np.array(refresh, dtype=_abi.CHUNK_DTYPE)
        refresh_max = int(refresh_np['n_alloc'].max())
    return LaunchPlan(rows_np, segs_np, refresh_np, refresh_max, block, info)
