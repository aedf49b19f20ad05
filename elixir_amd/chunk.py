"""Flat chunk storage: the one-process subset of the reference's chunk runtime that the optimizer
step reads and writes (``elixir/chunk/core/chunk.py``, ``group.py``).

A chunk stores a sequence of tensors back to back in one 1-D buffer.  Parameters live in a pair of
chunks with identical offsets: a low-precision chunk whose permanent ``shard`` doubles as the
gradient buffer at step time, and an fp32 chunk that holds the master weights
(``elixir/wrapper/module.py:104-133``).  On one process ``shard_size == chunk_size`` and
``shard_begin == 0``.

What is kept: the layout fields and rules (``append_tensor``, ``close_chunk``, ``valid_end``,
``tensors_info``, ``init_pair``), the landing of reduced gradients in the shard (``reduce_chunk``;
``land_chunks`` / ``land_tensors`` for many chunks in one launch) with the reduction flags
(``overflow``, ``l2_norm``, ``update_extra_reduce_info``) taken in the same pass, ``optim_update``,
the source copy of the gather and the release (``replicate`` / ``scatter`` on a caller-provided
block) including the deferred refresh of host-resident shards, and ``get_cpu_copy`` /
``load_tensors``.  Everything that touches chunk contents on the GPU runs on the HIP kernels.  What is
not here: the replicated-cache block pool, the collectives and the tensor state machine of the
forward/backward pass.
"""
import math
import weakref
from dataclasses import dataclass
from enum import Enum
from typing import Dict, List, Optional

import numpy as np
import torch

from . import _abi


class ChunkFullError(Exception):
    pass


class TensorState(Enum):
    FREE = 0
    COMPUTE = 1
    HOLD = 2
    HOLD_AFTER_BWD = 3
    READY_FOR_REDUCE = 4


@dataclass
class TensorInfo:
    state: TensorState
    fake_data: Optional[torch.Tensor]
    offset: int
    end: int


def gpu_device() -> torch.device:
    return torch.device('cuda', torch.cuda.current_device())


def kernel_device(tensors) -> torch.device:
    """The GPU whose kernels will touch these buffers.  Each must be device memory or pinned host
    memory (read and written in place over the host link); pageable host memory is refused."""
    device = None
    for t in tensors:
        if t.is_cuda:
            device = device or t.device
        elif not (torch.cuda.is_available() and t.is_pinned()):
            raise RuntimeError('the HIP kernels reach device memory and pinned host memory only: this shard lives in '
                               'pageable host memory (allocate it with cpu_pin_memory=True) or there is no GPU')
    return device or gpu_device()


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return {torch.float32: _abi.ELX_F32, torch.float16: _abi.ELX_F16, torch.bfloat16: _abi.ELX_BF16}[dtype]
    except KeyError:
        raise TypeError(f'chunks hold float32, float16 or bfloat16, not {dtype}') from None


class DeviceTable:
    """A numpy structured array and its copy in device memory."""

    def __init__(self, host: np.ndarray, device: torch.device):
        self.host = host
        self.dev = torch.from_numpy(host.view(np.uint8).reshape(-1).copy()).to(device)

    @property
    def ptr(self) -> int:
        return self.dev.data_ptr()

    def __len__(self):
        return len(self.host)


CACHED_STATS_WORKGROUPS = 1280    # whole launch, when the gradients are served from the memory-side cache


def stats_launch_blocks(n_valid_max: int, n_chunks: int = 1, cached: bool = False) -> int:
    """Workgroups per chunk for the stats pass: enough to fill 256 compute units several times
    over for large chunks, one per 16 Ki elements for small ones.  A set that the memory-side cache
    serves (``cached``: the launch reads it with ordinary loads) is read fastest by about five workgroups
    per compute unit in all -- the two chunks of GPT-2 small: 43 us with 384 to 896 workgroups per chunk,
    47 us with 1024 (every compute unit filled to its eight) and 46 us with 320."""
    blocks = int(max(1, min(1024, math.ceil(n_valid_max / 16384))))
    if cached:
        blocks = max(1, min(blocks, CACHED_STATS_WORKGROUPS // max(1, n_chunks)))
    return blocks


# The memory-side cache of the GPU holds 256 MiB.  A gradient set below this size is read by the stats pass
# with ordinary loads, so that the update launch right behind it finds the gradients there (step time
# -2 % to -5 % between 64 and 256 MiB of gradients); larger sets are read with non-temporal loads, which
# stream faster (a 2.6 GB set: 0.39 against 0.45 ms).  A landing launch follows the same rule with its
# stores (GPT-2 small: landing 0.145 -> 0.139 ms, the step behind it 0.573 -> 0.556 ms; the 2.95 GB of
# OPT-1.3B: landing 0.97 -> 1.00 ms with ordinary stores, so they stay non-temporal).
KEEP_GRADS_CACHED_BELOW = 256 << 20


def keep_grads_cached(chunk_rows: np.ndarray, grad_dtype: int) -> bool:
    """Whether the gradients the stats launch over ``chunk_rows`` reads fit the memory-side cache."""
    esize = 4 if grad_dtype == _abi.ELX_F32 else 2
    return int(chunk_rows['n_valid'].sum()) * esize <= KEEP_GRADS_CACHED_BELOW


def launch_grad_stats(chunk_rows: np.ndarray, grad_dtype: int, device: torch.device,
                      table: Optional[DeviceTable] = None, workspace: Optional[Dict] = None) -> torch.Tensor:
    """Enqueues the stats pass for the chunks described by ``chunk_rows`` (host table, only grad /
    n_alloc / n_valid are read) on the current stream and returns the device bytes that will hold
    the per-chunk ElxStats records."""
    n = len(chunk_rows)
    if table is None:
        table = DeviceTable(chunk_rows, device)
    cached = keep_grads_cached(chunk_rows, grad_dtype)
    bpc = stats_launch_blocks(int(chunk_rows['n_valid'].max()), n, cached)
    aligned = bool(np.all(chunk_rows['grad'] % 16 == 0))
    if workspace is None:
        workspace = {}
    need = (n * bpc + n) * _abi.STATS_DTYPE.itemsize
    buf = workspace.get('stats')
    if buf is None or buf.numel() < need or buf.device != device:
        buf = torch.empty(need, dtype=torch.uint8, device=device)
        workspace['stats'] = buf
    workspace['stats_table'] = table    # keep the table alive until the launch has run
    d_partials = buf.data_ptr()
    d_stats = d_partials + n * bpc * _abi.STATS_DTYPE.itemsize
    stream = torch.cuda.current_stream(device).cuda_stream
    _abi.grad_stats_mt(table.ptr, n, grad_dtype, bpc, d_partials, d_stats, not aligned, stream, keep_cached=cached)
    return buf[n * bpc * _abi.STATS_DTYPE.itemsize:need]


def read_grad_stats(dev_records: torch.Tensor) -> np.ndarray:
    """One blocking device-to-host copy of 16 bytes per chunk."""
    return dev_records.cpu().numpy().view(_abi.STATS_DTYPE).copy()


def run_grad_stats(chunk_rows: np.ndarray, grad_dtype: int, device: torch.device, table: Optional[DeviceTable] = None,
                   workspace: Optional[Dict] = None) -> np.ndarray:
    """Stats pass + readback: the per-chunk ElxStats records on the host."""
    return read_grad_stats(launch_grad_stats(chunk_rows, grad_dtype, device, table, workspace))


def l2_norm_from_sumsq(sumsq: float) -> float:
    """chunk.py:218-221 -- the reference takes the norm as an fp32 scalar and squares it in a
    Python float: ``valid.float().norm(2).item() ** 2``."""
    return float(np.float32(math.sqrt(sumsq)))**2


LAND_BLOCKS_PER_CU = 0    # 0: the library default


class StatsArena:
    """Device ElxStats records that landing launches leave behind, one slot per chunk, so that the
    optimizer step can fetch the flags of all chunks with one device-to-host copy.  Slots are handed
    out in consecutive runs (the chunks of one landing sit side by side) and go back to the arena
    when their chunk is given another slot or is garbage-collected."""
    CAPACITY = 65535    # the chunks one launch can take: a set never needs more slots than that (1 MiB per device)
    _arenas: Dict[torch.device, 'StatsArena'] = {}

    def __init__(self, device: torch.device):
        self.device = device
        self.itemsize = _abi.STATS_DTYPE.itemsize
        self.buf = torch.zeros(self.CAPACITY * self.itemsize, dtype=torch.uint8, device=device)
        self.used = np.zeros(self.CAPACITY, dtype=bool)

    @classmethod
    def get(cls, device: torch.device) -> 'StatsArena':
        device = torch.device(device)
        arena = cls._arenas.get(device)
        if arena is None:
            arena = cls._arenas[device] = StatsArena(device)
        return arena

    def new_slots(self, count: int) -> int:
        """First index of ``count`` consecutive free slots (first fit), now taken."""
        assert count >= 1
        if count <= self.CAPACITY:
            filled = np.concatenate(([0], np.cumsum(self.used)))
            runs = np.flatnonzero(filled[count:] == filled[:-count])    # windows without a used slot
            if len(runs):
                first = int(runs[0])
                self.used[first:first + count] = True
                return first
        raise RuntimeError(f'no run of {count} free stats slots on {self.device} '
                           f'({int(self.used.sum())} of {self.CAPACITY} in use)')

    def release(self, slot: int) -> None:
        self.used[slot] = False

    def assign(self, chunks: List['Chunk']) -> None:
        """Gives the chunks of one landing consecutive slots in list order, keeping the ones they hold
        when those already are."""
        slots = [c._stats_slot for c in chunks]
        if slots[0] is not None and all(b is not None and b == a + 1 for a, b in zip(slots, slots[1:])) \
                and all(c._stats_home[0] is self for c in chunks):
            return
        first = self.new_slots(len(chunks))
        for i, c in enumerate(chunks):
            c._take_stats_slot(self, first + i)

    def pin(self, chunks: List['Chunk']) -> None:
        """Gives the chunks consecutive slots in list order for as long as they live (an optimizer does this
        for its parameter chunks, in chunk order): in whatever order and grouping they land afterwards --
        one launch per chunk from the hooks of backward, last chunk first -- their records end up side by
        side, where one launch of the step folds them."""
        if all(c._stats_pinned and c._stats_home[0] is self for c in chunks) and \
                all(b._stats_slot == a._stats_slot + 1 for a, b in zip(chunks, chunks[1:])):
            return
        first = self.new_slots(len(chunks))
        for i, c in enumerate(chunks):
            c._take_stats_slot(self, first + i)
            c._stats_pinned = True

    def runs(self, chunks: List['Chunk']) -> List[List['Chunk']]:
        """The chunks of one landing cut into runs that one launch each can serve (a launch writes its
        records into consecutive slots, in list order).  A pinned chunk keeps its slot, and a run ends
        where the next chunk's pinned slot does not follow; chunks without a pinned slot get consecutive
        ones from ``assign``."""
        runs: List[List['Chunk']] = []
        for c in chunks:
            pinned = c._stats_pinned and c._stats_home[0] is self
            if runs:
                prev = runs[-1][-1]
                prev_pinned = prev._stats_pinned and prev._stats_home[0] is self
                if pinned == prev_pinned and (not pinned or c._stats_slot == prev._stats_slot + 1):
                    runs[-1].append(c)
                    continue
            runs.append([c])
        for run in runs:
            if not (run[0]._stats_pinned and run[0]._stats_home[0] is self):
                self.assign(run)
        return runs

    def ptr(self, slot: int) -> int:
        return self.buf.data_ptr() + slot * self.itemsize

    def read(self, lo: int, hi: int) -> np.ndarray:
        """Slots [lo, hi) on the host: one blocking copy."""
        return self.buf[lo * self.itemsize:hi * self.itemsize].cpu().numpy().view(_abi.STATS_DTYPE).copy()


def _release_stats_home(home: list) -> None:
    """Finalizer of a chunk: its slot, if it still holds one, goes back to its arena."""
    arena, slot = home
    if arena is not None and slot is not None:
        arena.release(slot)


def land_chunks(chunks: List['Chunk'], payloads: List[torch.Tensor], mul: float = 1.0) -> None:
    """Fused gradient landing for a list of chunks in ONE launch: ``payloads[i]`` (``shard_size``
    elements: the slice of the reduced payload that belongs to the shard; the chunk's dtype, or fp32)
    overwrites ``chunks[i].shard`` while the overflow flag and the sum of squares of what now sits in
    ``shard[:valid_end]`` are left in the chunk's slot of the device arena.  Nothing is read back
    here; ``Chunk.overflow`` / ``Chunk.l2_norm`` (or the optimizer step, for all chunks at once)
    fetch the records when they are needed.  Replaces chunk.py:309-315 + 345-356."""
    if not chunks:
        return
    device = chunks[0].shard_device
    if device.type != 'cuda':
        raise RuntimeError('gradients land through the HIP kernels: shards must be on the GPU')
    dst_code = dtype_code(chunks[0].chunk_dtype)
    src_code = dtype_code(payloads[0].dtype)
    for c, pl in zip(chunks, payloads):
        assert not c.is_init
        assert c.shard_device == device and pl.device == device and pl.is_contiguous()
        assert dtype_code(c.chunk_dtype) == dst_code and dtype_code(pl.dtype) == src_code
        assert pl.numel() == c.shard_size, 'the payload slice must cover the shard'
    arena = StatsArena.get(device)
    payload_of = {c: pl for c, pl in zip(chunks, payloads)}
    for run in arena.runs(list(chunks)):
        _land_chunks_run(arena, run, [payload_of[c] for c in run], src_code, dst_code, mul)


def _mark_landed(chunks: List['Chunk'], device: torch.device) -> None:
    """The records of these chunks are on their way: an event behind the launch, on its stream."""
    stream = torch.cuda.current_stream(device)
    landed = torch.cuda.Event()
    landed.record(stream)
    for c in chunks:
        c._overflow = False
        c._l2_norm = None
        c._stats_fresh = False
        c._stats_pending = True
        c._stats_event = landed
        c._stats_stream = stream.cuda_stream


def _land_chunks_run(arena: 'StatsArena', chunks: List['Chunk'], payloads: List[torch.Tensor], src_code: int,
                     dst_code: int, mul: float) -> None:
    """One launch: the records of ``chunks`` are consecutive slots of ``arena``."""
    device = chunks[0].shard_device
    rows = np.zeros(len(chunks), dtype=_abi.CHUNK_DTYPE)
    for i, (c, pl) in enumerate(zip(chunks, payloads)):
        rows[i]['grad'] = pl.data_ptr()
        rows[i]['lowp_out'] = c.shard.data_ptr()
        rows[i]['n_alloc'] = c.shard_size
        rows[i]['n_valid'] = c.n_valid
    aligned = bool(np.all(rows['grad'] % 16 == 0) and np.all(rows['lowp_out'] % 16 == 0))
    bpr = _abi.check_land_rows(rows, None, src_code, dst_code)
    ws = chunks[0]._workspace
    need = _abi.land_workspace_records(len(rows), bpr) * arena.itemsize
    buf = ws.get('land')
    if buf is None or buf.numel() < need:
        buf = ws['land'] = torch.empty(need, dtype=torch.uint8, device=device)
    cached = ws.get('land_table')
    if cached is None or not np.array_equal(cached.host, rows):
        cached = ws['land_table'] = DeviceTable(rows, device)
    stream = torch.cuda.current_stream(device).cuda_stream
    _abi.land_grads_mt(cached.ptr, len(rows), src_code, dst_code, float(np.float32(mul)), bpr, buf.data_ptr(),
                       arena.ptr(chunks[0]._stats_slot), aligned, stream, LAND_BLOCKS_PER_CU,
                       keep_cached=keep_grads_cached(rows, dst_code))
    _mark_landed(chunks, device)


LAND_MAX_BLOCK_TILES = 2048    # tiles per row where a launch over long tensors was measured to stream best
LAND_MAX_ROWS = 32768          # the grid's y extent must stay below 65536
LAND_IDLE_ALLOWED = 0.025      # share of workgroups without work that a larger block may cost


def _land_block_elems(counts, tile: int) -> int:
    """Rows of a per-tensor landing are blocks of a power-of-two number of tiles.  The launch is a grid of
    (tiles of the longest row, rows), so every row shorter than that leaves workgroups that find no work:
    with blocks of 2048 tiles the 148 gradients of GPT-2 small (768 ... 38.6 M elements) make 327,680
    workgroups for 65,536 tiles of work and the launch runs at half its speed (178 us; 99 us with blocks of
    16 tiles, 103 us for the same shards landed from whole payloads).  Short blocks cost nothing on the
    device -- OPT-1.3B: 1.007 / 0.950 / 0.917 / 0.909 ms with 2048 / 512 / 128 / 64 tiles, LLaMA-7B 4.317 /
    4.279 / 4.303 ms with 2048 / 512 / 128 -- only host time when the table is first built.  ``counts``: the
    element counts of the pieces.  Picks the largest block, up to ``LAND_MAX_BLOCK_TILES`` tiles, whose launch
    has at most ``LAND_IDLE_ALLOWED`` idle workgroups (failing that, the block with the fewest
    workgroups) among those that keep the launch within ``LAND_MAX_ROWS`` rows; a set too large for that
    gets longer blocks."""
    counts = np.asarray(counts, dtype=np.int64)
    tiles = -(-counts // tile)
    work = int(tiles.sum())
    longest = int(tiles.max()) if len(tiles) else 1
    block_tiles = LAND_MAX_BLOCK_TILES
    while int((-(-counts // (block_tiles * tile))).sum()) > LAND_MAX_ROWS:
        block_tiles <<= 1
    if block_tiles > LAND_MAX_BLOCK_TILES:
        return block_tiles * tile
    best, best_wgs = block_tiles, None
    while block_tiles >= 8:
        rows = int((-(-counts // (block_tiles * tile))).sum())
        if rows > LAND_MAX_ROWS:
            break
        wgs = rows * min(block_tiles, longest)
        if wgs <= (1.0 + LAND_IDLE_ALLOWED) * work:
            return block_tiles * tile
        if best_wgs is None or wgs < best_wgs:
            best, best_wgs = block_tiles, wgs
        block_tiles >>= 1
    return best * tile


def land_rows(pieces, n_slots: int, block: int, ssize: int, dsize: int):
    """The row table of a per-tensor landing.  ``pieces``: (slot, source address or 0 for zeros,
    destination address, element count), the pieces of one slot consecutive and slots ascending.
    Every piece becomes ceil(count / block) rows.  Returns (rows, slot_offsets) where the rows
    [slot_offsets[s], slot_offsets[s + 1]) belong to slot s."""
    per_slot = np.zeros(n_slots + 1, dtype=np.int64)
    if not pieces:
        return np.zeros(0, dtype=_abi.CHUNK_DTYPE), per_slot.astype(np.uint32)
    slot, src, dst, count = (np.array(col, dtype=np.uint64) for col in zip(*pieces))
    n_rows = (count + np.uint64(block - 1)) // np.uint64(block)
    first_row = np.concatenate(([0], np.cumsum(n_rows)[:-1])).astype(np.uint64)
    total = int(n_rows.sum())
    piece = np.repeat(np.arange(len(pieces)), n_rows.astype(np.int64))
    start = (np.arange(total, dtype=np.uint64) - first_row[piece]) * np.uint64(block)    # element offset in the piece
    rows = np.zeros(total, dtype=_abi.CHUNK_DTYPE)
    has_src = src[piece] != 0
    rows['grad'] = np.where(has_src, src[piece] + start * np.uint64(ssize), 0)
    rows['lowp_out'] = dst[piece] + start * np.uint64(dsize)
    rows['n_alloc'] = np.minimum(np.uint64(block), count[piece] - start)
    rows['n_valid'] = np.where(has_src, rows['n_alloc'], 0)
    np.add.at(per_slot, slot.astype(np.int64) + 1, n_rows.astype(np.int64))
    return rows, np.cumsum(per_slot).astype(np.uint32)


def land_tensors(chunks: List['Chunk'], grad_of, mul: float = 1.0) -> None:
    """Lands chunks straight from the per-tensor gradients, in ONE launch for the whole list:
    ``grad_of(tensor)`` is the gradient of a tensor of the chunk (contiguous, on the shard's device,
    all of one dtype: the chunk's or fp32).  Every gradient is copied (cast) into its slice of the
    shard, what no tensor covers is zeroed, and the flags of each chunk are left in its slot of the
    device arena, as ``land_chunks`` leaves them.  Replaces the per-parameter copies of
    chunk.py:386-393 / module.py:177-190, the intermediate payload, and chunk.py:309-315 + 345-356.

    Each gradient is listed as rows of equal blocks (the last one shorter); a slice whose byte
    offset in the shard is not a multiple of 16 is moved element by element by its workgroups."""
    if not chunks:
        return
    device = chunks[0].shard_device
    if device.type != 'cuda':
        raise RuntimeError('gradients land through the HIP kernels: shards must be on the GPU')
    dst_dtype = chunks[0].chunk_dtype
    dst_code = dtype_code(dst_dtype)
    dsize = chunks[0].shard.element_size()
    src_dtype = None
    pieces = []    # (chunk index, src address or 0, begin in the shard, element count)
    for ci, c in enumerate(chunks):
        assert not c.is_init and c.shard_device == device and c.chunk_dtype == dst_dtype
        covered = 0
        for tensor, info in sorted(c.tensors_info.items(), key=lambda kv: kv[1].offset):
            g = grad_of(tensor)
            assert g is not None, 'every tensor of a chunk needs a gradient before the chunk can land'
            assert g.device == device and g.is_contiguous() and g.numel() == info.end - info.offset
            src_dtype = src_dtype or g.dtype
            assert g.dtype == src_dtype, 'all gradients of one landing must have one dtype'
            begin, end = max(info.offset, c.shard_begin) - c.shard_begin, min(info.end, c.shard_end) - c.shard_begin
            if begin >= end:
                continue
            if begin > covered:
                pieces.append((ci, 0, covered, begin - covered))
            pieces.append((ci, g.data_ptr() + (begin + c.shard_begin - info.offset) * g.element_size(), begin, end - begin))
            covered = end
        if covered < c.shard_size:
            pieces.append((ci, 0, covered, c.shard_size - covered))
    src_code = dtype_code(src_dtype if src_dtype is not None else dst_dtype)
    ssize = 4 if src_code == _abi.ELX_F32 else 2
    tile = _abi.land_tile_elems(src_code)
    arena = StatsArena.get(device)
    index_of = {c: ci for ci, c in enumerate(chunks)}
    for run in arena.runs(list(chunks)):
        first = index_of[run[0]]
        mine = [(ci - first, src, chunks[ci].shard.data_ptr() + begin * dsize, count)
                for ci, src, begin, count in pieces if first <= ci < first + len(run)]
        _land_tensors_run(arena, run, mine, tile, src_code, dst_code, ssize, dsize, mul)


LAND_TABLES_KEPT = 4    # device copies of row tables kept per chunk (gradient buffers tend to come back at the same addresses)


def _land_tensors_run(arena: 'StatsArena', chunks: List['Chunk'], pieces, tile: int, src_code: int, dst_code: int,
                      ssize: int, dsize: int, mul: float) -> None:
    """One launch: the records of ``chunks`` are consecutive slots of ``arena``; ``pieces`` as for
    ``land_rows``, slots counted from the first chunk of the run."""
    device = chunks[0].shard_device
    ws = chunks[0]._workspace
    # The tables of a landing are the same from step to step whenever the gradients come back at the same
    # addresses: they are kept, device copies included, under the list of pieces they were built from (building
    # them again costs the host a millisecond per 20,000 rows, and an upload from pageable memory makes it wait
    # for the stream).
    tables = ws.setdefault('land_tables', {})
    key = (tuple(pieces), tuple(c.chunk_id for c in chunks), src_code, dst_code)
    kept = tables.get(key)
    if kept is None:
        block = _land_block_elems([count for _, _, _, count in pieces], tile)
        rows, slot_offsets = land_rows(pieces, len(chunks), block, ssize, dsize)
        if len(rows) > 65535:
            raise RuntimeError(f'{len(rows)} rows in one landing launch: land fewer chunks at a time')
        bpr = _abi.check_land_rows(rows, slot_offsets, src_code, dst_code)
        if len(tables) >= LAND_TABLES_KEPT:
            tables.pop(next(iter(tables)))
        kept = tables[key] = (DeviceTable(rows, device), torch.from_numpy(slot_offsets.view(np.int32).copy()).to(device),
                              bpr)
    table, offsets, bpr = kept
    n_rows = len(table)
    need = _abi.land_workspace_records(n_rows, bpr, len(chunks)) * arena.itemsize
    buf = ws.get('land')
    if buf is None or buf.numel() < need:
        buf = ws['land'] = torch.empty(need, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    _abi.land_grads_mt(table.ptr, n_rows, src_code, dst_code, float(np.float32(mul)), bpr, buf.data_ptr(),
                       arena.ptr(chunks[0]._stats_slot), True, stream, LAND_BLOCKS_PER_CU,
                       d_slot_offsets=offsets.data_ptr(), n_slots=len(chunks),
                       keep_cached=sum(c.n_valid for c in chunks) * dsize <= KEEP_GRADS_CACHED_BELOW)
    _mark_landed(chunks, device)


def resolve_pending_stats(chunks: List['Chunk']) -> None:
    """Fetches the landing records of every chunk in the list that has one outstanding: one copy
    per device."""
    by_device: Dict[torch.device, List['Chunk']] = {}
    for c in chunks:
        if c._stats_pending:
            by_device.setdefault(c.shard_device, []).append(c)
    for device, pending in by_device.items():
        # the landing may have been enqueued on another stream than the one the copy below uses
        stream = torch.cuda.current_stream(device)
        for event in {c._stats_event for c in pending
                      if c._stats_event is not None and c._stats_stream != stream.cuda_stream}:
            stream.wait_event(event)
        lo = min(c._stats_slot for c in pending)
        hi = max(c._stats_slot for c in pending) + 1
        records = StatsArena.get(device).read(lo, hi)
        for c in pending:
            rec = records[c._stats_slot - lo]
            c._stats_pending = False
            c._stats_event = None
            c._apply_stats(bool(rec['overflow']), float(rec['sumsq']))


class Chunk:
    """A continuous memory block that stores a sequence of tensors (chunk.py:27-139).

    args:
        rcache: unused here (the replicated cache belongs to the forward/backward pass)
        chunk_size: number of elements
        chunk_dtype: element type
        process_group: must be None or a group of size 1
        temp_device: device of the temporary full chunk that exists while tensors are appended
        shard_device: device of the permanent shard (default: the current GPU, CPU without one)
    """
    total_count = 0

    def __init__(self,
                 rcache=None,
                 chunk_size: int = 0,
                 chunk_dtype: torch.dtype = torch.float,
                 process_group=None,
                 temp_device: Optional[torch.device] = None,
                 shard_device: Optional[torch.device] = None,
                 rcache_fused: bool = False,
                 cpu_pin_memory: bool = False) -> None:
        self.chunk_id: int = Chunk.total_count
        Chunk.total_count += 1
        self.rcache = rcache

        self.chunk_size: int = chunk_size
        self.chunk_dtype: torch.dtype = chunk_dtype
        self.utilized_size: int = 0

        self.torch_pg = process_group
        self.pg_size: int = 1
        self.pg_rank: int = 0
        if process_group is not None:
            import torch.distributed as dist
            if dist.get_world_size(process_group) != 1:
                raise NotImplementedError('this build keeps whole chunks on one GPU (process group of size 1)')
        assert chunk_size % self.pg_size == 0

        self.shard_size: int = chunk_size // self.pg_size
        self.shard_begin: int = self.shard_size * self.pg_rank
        self.shard_end: int = self.shard_begin + self.shard_size
        self.valid_end: int = self.shard_size + 1    # set to an illegal number

        self.rcb = None
        self.rcache_fused: bool = rcache_fused
        self.is_replica: bool = True

        default_device = gpu_device() if torch.cuda.is_available() else torch.device('cpu')
        temp_device = torch.device(temp_device) if temp_device is not None else default_device
        shard_device = torch.device(shard_device) if shard_device is not None else default_device
        # keep all elements to zero: the padding of every shard starts as zero
        self.chunk_temp: Optional[torch.Tensor] = None
        self._temp_device = temp_device
        self._meta_only = False
        pin_flag = cpu_pin_memory and shard_device.type == 'cpu'
        self.shard: torch.Tensor = torch.empty(self.shard_size, dtype=chunk_dtype, device=shard_device,
                                               pin_memory=pin_flag)
        self._is_init = True

        self.tensors_info: Dict[torch.Tensor, TensorInfo] = {}
        self.num_tensors: int = 0
        self.tensor_state_cnter: Dict[TensorState, int] = {state: 0 for state in TensorState}

        self.paired_chunk: Optional['Chunk'] = None
        # if this chunk is synchronized with the optimizer, the flag is True
        self.optim_sync_flag = True
        # whether to record l2 norm for the gradient clipping calculation
        self.l2_norm_flag = False
        # squared l2 norm / overflow of the reduced gradients; both are properties that first fetch
        # the record a fused landing left on the device, if one is outstanding
        self._l2_norm: Optional[float] = None
        self._overflow = False
        # True once overflow / l2_norm describe the gradients that sit in the shard now
        self._stats_fresh = False
        self._stats_slot: Optional[int] = None    # this chunk's record in the device arena
        self._stats_pinned = False                # the slot is this chunk's for good (StatsArena.pin)
        self._stats_home = [None, None]           # [arena, slot], shared with the finalizer that frees the slot
        weakref.finalize(self, _release_stats_home, self._stats_home)
        self._stats_pending = False               # a landing launch has written it, nobody has read it
        self._stats_event = None                  # recorded behind that launch, on its stream
        self._stats_stream = None                 # that stream's handle
        self._workspace: Dict = {}

    # ------------------------------------------------------------------ properties

    @property
    def is_init(self) -> bool:
        return self._is_init

    @property
    def overflow(self) -> bool:
        if self._stats_pending:
            resolve_pending_stats([self])
        return self._overflow

    @overflow.setter
    def overflow(self, value: bool) -> None:
        self._overflow = bool(value)

    @property
    def l2_norm(self) -> Optional[float]:
        if self._stats_pending:
            resolve_pending_stats([self])
        return self._l2_norm

    @l2_norm.setter
    def l2_norm(self, value: Optional[float]) -> None:
        self._l2_norm = value

    def _take_stats_slot(self, arena: 'StatsArena', slot: int) -> None:
        """This chunk's record moves to ``slot`` of ``arena``; the slot it held goes back."""
        old_arena, old_slot = self._stats_home
        if old_arena is not None and old_slot is not None:
            old_arena.release(old_slot)
        self._stats_slot = slot
        self._stats_pinned = False
        self._stats_home[0], self._stats_home[1] = arena, slot

    def invalidate_stats(self) -> None:
        """The shard was written behind the chunk's back: forget flags and outstanding records."""
        self._stats_pending = False
        self._stats_event = None
        self._stats_fresh = False
        self._overflow = False
        self._l2_norm = None

    @property
    def shard_device(self) -> torch.device:
        return self.shard.device

    @property
    def payload(self) -> torch.Tensor:
        if self.is_init and self.chunk_temp is not None:
            return self.chunk_temp
        return self.shard

    @property
    def n_valid(self) -> int:
        """Number of shard elements that hold tensor data: ``shard[:valid_end]`` (chunk.py:352)."""
        return min(self.valid_end, self.shard_size)

    @property
    def memory_usage(self) -> Dict[str, int]:
        memo = self.shard_size * self.shard.element_size()
        cuda = memo if self.shard_device.type == 'cuda' else 0
        cpu = memo if self.shard_device.type == 'cpu' else 0
        if self.chunk_temp is not None:
            t = self.chunk_size * self.chunk_temp.element_size()
            if self.chunk_temp.device.type == 'cuda':
                cuda += t
            else:
                cpu += t
        return dict(cuda=cuda, cpu=cpu)

    # ------------------------------------------------------------------ building

    def append_tensor(self, tensor: torch.Tensor):
        """chunk.py:223-247.  Tensors are packed back to back with no alignment padding.  A tensor
        on the ``meta`` device only reserves its range (its values are produced in place later)."""
        assert self.is_init
        assert tensor.dtype == self.chunk_dtype

        new_utilized_size = self.utilized_size + tensor.numel()
        if new_utilized_size > self.chunk_size:
            raise ChunkFullError

        if tensor.device.type != 'meta':
            if self.chunk_temp is None:
                assert not self._meta_only, 'a chunk holds either real or meta tensors'
                self.chunk_temp = torch.zeros(self.chunk_size, dtype=self.chunk_dtype, device=self._temp_device)
            self.chunk_temp[self.utilized_size:new_utilized_size].copy_(tensor.data.flatten())
            tensor.data = self.chunk_temp[self.utilized_size:new_utilized_size].view(tensor.shape)
        else:
            assert self.chunk_temp is None, 'a chunk holds either real or meta tensors'
            self._meta_only = True

        self.num_tensors += 1
        tensor_state = TensorState.HOLD
        self.tensor_state_cnter[tensor_state] += 1
        # a data-less stand-in that remembers the tensor's shape while its storage lives in the chunk
        fake_data = torch.empty(tensor.shape, dtype=tensor.dtype, device='meta')
        self.tensors_info[tensor] = TensorInfo(state=tensor_state, fake_data=fake_data, offset=self.utilized_size,
                                               end=new_utilized_size)
        self.utilized_size = new_utilized_size

    def close_chunk(self):
        """chunk.py:249-262: fix ``valid_end`` and move the data into the permanent shard."""
        assert self.is_init

        if self.utilized_size <= self.shard_begin:
            self.valid_end = 0
        elif self.utilized_size < self.shard_end:
            self.valid_end = self.utilized_size - self.shard_begin

        if self.chunk_temp is not None:
            for tensor, info in self.tensors_info.items():
                tensor.data = torch.empty(0, dtype=tensor.dtype, device=tensor.device)
            self.shard.copy_(self.chunk_temp[self.shard_begin:self.shard_end])
        else:
            self.shard.zero_()
        self.is_replica = False
        self.chunk_temp = None
        self._is_init = False

    def init_pair(self, friend_chunk: 'Chunk') -> None:
        if self.paired_chunk is None and friend_chunk.paired_chunk is None:
            self.paired_chunk = friend_chunk
            friend_chunk.paired_chunk = self
        else:
            assert self.paired_chunk is friend_chunk
            assert friend_chunk.paired_chunk is self

    def get_tensors(self) -> List[torch.Tensor]:
        return list(self.tensors_info.keys())

    def get_cpu_copy(self, only_rank_0: bool = False) -> List[torch.Tensor]:
        """chunk.py:426-447 on one process: a CPU copy of every tensor of the chunk, in order,
        shaped like the tensor."""
        assert not self.is_init
        return [self.shard[info.offset:info.end].view(info.fake_data.shape if info.fake_data is not None else t.shape)
                .cpu() for t, info in self.tensors_info.items()]

    def load_tensors(self, tensor_list: List[Optional[torch.Tensor]], only_rank_0: bool = False) -> None:
        """chunk.py:449-473 on one process: values for the tensors of the chunk, in order (None =
        keep), written into the shard."""
        assert not self.is_init
        assert len(tensor_list) == len(self.tensors_info)
        for info, load_tensor in zip(self.tensors_info.values(), tensor_list):
            if load_tensor is None:
                continue
            self.shard[info.offset:info.end].copy_(load_tensor.data.flatten())
        self.invalidate_stats()

    # ------------------------------------------------------------------ gradient landing and flags

    def set_overflow_flag(self, valid_tensor: Optional[torch.Tensor] = None) -> None:
        """chunk.py:214-216; here both flags come from one pass over ``shard[:valid_end]``."""
        assert not self._stats_pending and not self._overflow
        self._compute_stats()

    def set_l2_norm(self, valid_tensor: Optional[torch.Tensor] = None) -> None:
        assert not self._stats_pending and self._l2_norm is None, 'you are calculating the l2 norm twice'
        self._compute_stats()

    def _compute_stats(self) -> None:
        device = kernel_device([self.shard])
        blocks = stats_launch_blocks(self.n_valid)
        rec = _abi.STATS_DTYPE.itemsize
        buf = self._workspace.get('stats_one')
        if buf is None or buf.numel() < (blocks + 1) * rec or buf.device != device:
            buf = self._workspace['stats_one'] = torch.empty((blocks + 1) * rec, dtype=torch.uint8, device=device)
        _abi.grad_stats(self.shard.data_ptr(), dtype_code(self.chunk_dtype), self.n_valid, blocks, buf.data_ptr(),
                        buf.data_ptr() + blocks * rec, torch.cuda.current_stream(device).cuda_stream)
        stats = read_grad_stats(buf[blocks * rec:(blocks + 1) * rec])
        self._apply_stats(bool(stats['overflow'][0]), float(stats['sumsq'][0]))

    def _apply_stats(self, overflow: bool, sumsq: float) -> None:
        self._overflow = overflow
        if self.l2_norm_flag:
            self._l2_norm = l2_norm_from_sumsq(sumsq)
        self._stats_fresh = True

    def update_extra_reduce_info(self, block=None):
        """chunk.py:345-356: flags over the valid head of the reduced gradients.  On one process
        those are the first ``valid_end`` elements of the shard.  After a fused landing the record
        already exists on the device and is only fetched; otherwise one stats pass runs."""
        if self._stats_pending:
            resolve_pending_stats([self])
            return
        assert not self._overflow
        assert self._l2_norm is None, 'you are calculating the l2 norm twice'
        self._compute_stats()

    def reduce_chunk(self, payload: torch.Tensor, always_fp32: bool = False, sync: bool = True) -> None:
        """The tail of chunk.py:282-315 / 358-377 for a process group of size 1: the gradients that
        backward accumulated in ``payload`` (``chunk_size`` elements of the chunk's dtype, or fp32
        for a reduction carried out in fp32) overwrite the shard.  The copy and the flags are one
        launch; with ``sync`` the flags are fetched right away (as the reference's blocking
        ``.item()`` calls do), otherwise they stay on the device until somebody reads
        ``overflow`` / ``l2_norm`` or the optimizer step collects them for all chunks at once."""
        assert not self.is_init
        assert payload.numel() == self.chunk_size
        if self.shard_device.type == 'cuda':
            land_chunks([self], [payload[self.shard_begin:self.shard_end]])
        else:
            # a host-resident shard: the landing is a transfer, and no flags come with it
            self.shard.copy_(payload[self.shard_begin:self.shard_end])
            self.invalidate_stats()
        if sync:
            self.update_extra_reduce_info()

    # ------------------------------------------------------------------ low-precision refresh

    def optim_update(self) -> None:
        """Update the low-precision chunk from its fp32 chunk (chunk.py:403-421)."""
        assert self.paired_chunk is not None
        friend_chunk: Chunk = self.paired_chunk
        assert not friend_chunk.is_replica
        # gradient and optimizer should be on the same device
        assert self.shard_device.type == friend_chunk.shard_device.type

        if self.shard_device.type == 'cuda':
            _abi.writeback(friend_chunk.shard.data_ptr(), self.shard.data_ptr(), dtype_code(self.chunk_dtype),
                           self.shard_size, torch.cuda.current_stream(self.shard_device).cuda_stream)
            self.optim_sync_flag = True
        elif self.shard_device.type == 'cpu':
            # the refresh is deferred to the next gather of this chunk
            self.optim_sync_flag = False
        else:
            raise NotImplementedError

    # ------------------------------------------------------------------ gather source / release

    def _refresh_into(self, dst: torch.Tensor, master: torch.Tensor) -> None:
        """dst (device, this chunk's dtype) = round-to-nearest-even(master); ``master`` is device
        memory or pinned host memory, which the kernel reads in place over the host link."""
        assert dst.is_cuda and dst.is_contiguous() and dst.numel() == master.numel() == self.shard_size
        assert master.dtype == torch.float32 and master.is_contiguous()
        assert master.is_cuda or master.is_pinned(), 'the kernel can only read device or pinned host memory'
        _abi.writeback(master.data_ptr(), dst.data_ptr(), dtype_code(self.chunk_dtype), self.shard_size,
                       torch.cuda.current_stream(dst.device).cuda_stream)

    def replicate(self, payload: torch.Tensor) -> None:
        """chunk.py:264-270 + 475-482 on one process: fills this shard's slice of a replicated block
        (``chunk_size`` elements on the GPU) -- the source copy of the gather.  A shard that is in
        sync with its optimizer chunk is copied (a transfer when it lives on the host).  One whose
        refresh was deferred (``optim_sync_flag`` False: host-resident shards after an update) is
        produced from the fp32 optimizer shard in ONE pass: the cast kernel reads pinned host memory
        in place and writes the low-precision slice, without the fp32 staging copy on the GPU that
        ``optim_chunk.shard.to(gpu)`` + ``copy_`` would make.  An unpinned host shard is staged."""
        assert not self.is_init
        assert payload.is_cuda and payload.numel() == self.chunk_size and payload.dtype == self.chunk_dtype
        dst = payload[self.shard_begin:self.shard_end]
        if self.optim_sync_flag:
            dst.copy_(self.shard)
            return
        assert self.paired_chunk is not None, 'chunks should be paired before training'
        master = self.paired_chunk.shard
        if not (master.is_cuda or master.is_pinned()):
            master = master.to(payload.device)
        self._refresh_into(dst, master)

    def scatter(self, payload: torch.Tensor) -> None:
        """chunk.py:273-281 on one process: the block is released; a shard whose refresh was
        deferred takes the refreshed values from the block and is in sync again."""
        assert not self.is_init
        assert payload.numel() == self.chunk_size and payload.dtype == self.chunk_dtype
        if not self.optim_sync_flag:
            self.shard.copy_(payload[self.shard_begin:self.shard_end])
            self.optim_sync_flag = True

    # ------------------------------------------------------------------ misc

    def __hash__(self) -> int:
        return self.chunk_id

    def __lt__(self, other: object) -> bool:
        return self.chunk_id < other.chunk_id

    def __eq__(self, other: object) -> bool:
        return isinstance(other, Chunk) and self.chunk_id == other.chunk_id

    def __repr__(self):
        state = 'initialization' if self.is_init else 'scattered'
        return (f'Chunk {self.chunk_id}: state -> {state}, length: {self.chunk_size}, dtype: {self.chunk_dtype}, '
                f'tensors: {self.num_tensors}, utilized size: {self.utilized_size}, valid_end: {self.valid_end}, '
                f'shard device: {self.shard_device}')


class ChunkGroup:
    """Bookkeeping of a set of chunks (group.py:12-98): which chunk holds which tensor."""

    def __init__(self, rcache=None) -> None:
        self.rcache = rcache
        self.fused_chunks: set = set()
        self.float_chunks: set = set()
        self.ten_to_chunk: Dict[torch.Tensor, Chunk] = dict()

    def open_chunk(self, chunk_size: int, chunk_dtype: torch.dtype, process_group=None,
                   chunk_config: Optional[Dict] = None) -> Chunk:
        if chunk_config is None:
            chunk_config = {}
        return Chunk(rcache=self.rcache, chunk_size=chunk_size, chunk_dtype=chunk_dtype, process_group=process_group,
                     **chunk_config)

    def close_chunk(self, chunk: Chunk) -> bool:
        chunk.close_chunk()
        if chunk.rcache_fused:
            self.fused_chunks.add(chunk)
        else:
            self.float_chunks.add(chunk)
        for t in chunk.get_tensors():
            assert t not in self.ten_to_chunk
            self.ten_to_chunk[t] = chunk
        return True

    def inside_check(self, chunk: Chunk) -> None:
        if chunk.rcache_fused:
            assert chunk in self.fused_chunks
        else:
            assert chunk in self.float_chunks

    @property
    def all_chunks(self) -> List[Chunk]:
        return sorted(self.fused_chunks.union(self.float_chunks))
