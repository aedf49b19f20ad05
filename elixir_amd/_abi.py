"""ctypes binding of ``libelx_hip.so`` (declared in ``include/elx_abi.h``).

There is no CPU fallback: if the library has not been built, or a launch fails, the caller gets
an exception.  Tables are built on the host as numpy structured arrays whose layouts mirror the
C structs (the sizes are checked against the loaded library).
"""
import ctypes
import os
from typing import Optional

import numpy as np

ELX_ABI_VERSION = 3
ELX_F32, ELX_F16, ELX_BF16, ELX_NONE = 0, 1, 2, -1
ELX_FLAG_SCALAR_ONLY = 1
ELX_FLAG_KEEP_CACHED = 2
ELX_FLAG_KEEP_STATE_CACHED = 4
ELX_E_NULL, ELX_E_DTYPE, ELX_E_ALIGN, ELX_E_RANGE, ELX_E_ORDER, ELX_E_TILES, ELX_E_SIZE, ELX_E_STATE = -1, -2, -3, -4, -5, -6, -7, -8
MAX_ARG_HYPERS = 32    # hyper records that ride in the arguments of an update launch (elx_adam_step_put_mt)
ELX_HYPER_L2 = 1
ELX_HYPER_LERP_FROM_G = 2

CHUNK_DTYPE = np.dtype([('grad', '<u8'), ('lowp_out', '<u8'), ('master', '<u8'), ('m', '<u8'), ('v', '<u8'),
                        ('n_alloc', '<u8'), ('n_valid', '<u8'), ('tile_begin', '<u8'), ('seg_begin', '<u4'),
                        ('seg_end', '<u4')])
SEG_DTYPE = np.dtype([('begin', '<u8'), ('end', '<u8'), ('hyper', '<u4'), ('reserved', '<u4')])
HYPER_DTYPE = np.dtype([('decay_mul', '<f4'), ('l2_wd', '<f4'), ('lerp_w', '<f4'), ('beta2', '<f4'), ('omb2', '<f4'),
                        ('bc2_sqrt', '<f4'), ('eps', '<f4'), ('neg_step', '<f4'), ('flags', '<u4'),
                        ('gate_div_scale', '<f4'), ('gate_inv_scale', '<f4'), ('gate', '<u4')])
STATS_DTYPE = np.dtype([('sumsq', '<f8'), ('overflow', '<u4'), ('reserved', '<u4')])
DECISION_DTYPE = np.dtype([('div_scale', '<f4'), ('inv_scale', '<f4'), ('mode', '<u4'), ('skip', '<u4'),
                           ('total_norm', '<f8'), ('combined_scale', '<f8')])

STEP_CTL_DTYPE = np.dtype([('loss_scale', '<f8'), ('max_norm', '<f8'), ('clipping', '<u4'), ('n_hypers', '<u4'),
                           ('seq', '<u8')])
STEP_REPORT_DTYPE = np.dtype([('div_scale', '<f4'), ('inv_scale', '<f4'), ('mode', '<u4'), ('skip', '<u4'),
                              ('total_norm', '<f8'), ('combined_scale', '<f8'), ('seq', '<u8'), ('n_chunks', '<u4'),
                              ('status', '<i4')])

LIB_NAME = 'libelx_hip.so'
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

EXPORTS = ('elx_version', 'elx_strerror', 'elx_tile_elems', 'elx_sizeof_chunk', 'elx_sizeof_seg', 'elx_sizeof_hyper',
           'elx_sizeof_stats', 'elx_sizeof_decision', 'elx_check_tables', 'elx_grad_stats_mt', 'elx_adam_step_mt',
           'elx_decide', 'elx_adam_step_gated_mt', 'elx_writeback_mt', 'elx_refresh_piece_elems', 'elx_writeback',
           'elx_grad_stats', 'elx_land_grads_mt', 'elx_check_land_rows', 'elx_land_max_blocks', 'elx_land_tile_elems',
           'elx_land_fold_blocks', 'elx_grad_stats_mt_static', 'elx_static_partials', 'elx_grad_partials_mt',
           'elx_finish_decide', 'elx_sizeof_step_ctl', 'elx_sizeof_step_report', 'elx_max_ctl_hypers', 'elx_put_hypers',
           'elx_adam_step_put_mt', 'elx_source_sha', 'elx_unscale_mode', 'elx_occupancy_lds_bytes', 'elx_finish_decide_rows')

# what the validators' own build (the host-only source under sanitizers) exports
HOST_EXPORTS = ('elx_check_tables', 'elx_check_land_rows', 'elx_tile_elems', 'elx_land_tile_elems', 'elx_land_max_blocks',
                'elx_unscale_mode', 'elx_occupancy_lds_bytes', 'elx_source_sha')

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc')
_HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'include', 'elx_abi.h')


def source_files():
    """The files a build of the library is made from, in the order their digest is taken."""
    files = [os.path.join(_CSRC, f) for f in sorted(os.listdir(_CSRC)) if f.endswith(('.hip', '.cpp', '.h'))]
    return files + [_HEADER]


def source_sha16() -> str:
    """First 16 hex digits of the SHA-256 over the library's sources as they are now."""
    import hashlib
    h = hashlib.sha256()
    for path in source_files():
        h.update(os.path.basename(path).encode() + b'\0')
        with open(path, 'rb') as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def built_source_sha(lib_path: str) -> str:
    """The digest a built library carries ('' when it has none)."""
    try:
        L = ctypes.CDLL(lib_path)
        L.elx_source_sha.restype = ctypes.c_char_p
        L.elx_source_sha.argtypes = []
        return (L.elx_source_sha() or b'').decode()
    except (OSError, AttributeError):
        return ''


class ElxError(RuntimeError):
    """A call into libelx_hip.so returned a non-zero code."""

    def __init__(self, func: str, code: int, text: str):
        super().__init__(f'{func} failed with code {code}: {text}')
        self.func = func
        self.code = code


_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise loudly when it is missing or does not match this binding."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f'{LIB_PATH} is missing: the HIP extension has not been built. '
                           f'Run `python -m elixir_amd.build` (needs hipcc); there is no CPU fallback.')
    L = ctypes.CDLL(LIB_PATH)
    u32, u64, vp, cint, flt = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.elx_version.restype = cint
    L.elx_version.argtypes = []
    L.elx_strerror.restype = ctypes.c_char_p
    L.elx_strerror.argtypes = [cint]
    for name in ('elx_tile_elems', 'elx_sizeof_chunk', 'elx_sizeof_seg', 'elx_sizeof_hyper', 'elx_sizeof_stats',
                 'elx_sizeof_decision', 'elx_refresh_piece_elems', 'elx_land_max_blocks', 'elx_land_fold_blocks',
                 'elx_static_partials', 'elx_sizeof_step_ctl', 'elx_sizeof_step_report', 'elx_max_ctl_hypers'):
        getattr(L, name).restype = u32
        getattr(L, name).argtypes = []
    L.elx_source_sha.restype = ctypes.c_char_p
    L.elx_source_sha.argtypes = []
    _bind_host(L)
    L.elx_grad_stats_mt.restype = cint
    L.elx_grad_stats_mt.argtypes = [vp, u32, cint, u32, vp, vp, cint, vp]
    L.elx_grad_partials_mt.restype = cint
    L.elx_grad_partials_mt.argtypes = [vp, u32, cint, u32, vp, cint, vp]
    L.elx_finish_decide.restype = cint
    L.elx_finish_decide.argtypes = [vp, u32, u32, vp, vp, vp, u32, vp, vp, vp, vp]
    L.elx_finish_decide_rows.restype = cint
    L.elx_finish_decide_rows.argtypes = [vp, u32, u32, vp, vp, vp, u32, vp, vp, vp, vp, vp, u32, vp, vp]
    L.elx_adam_step_put_mt.restype = cint
    L.elx_adam_step_put_mt.argtypes = [vp, u32, vp, u32, vp, vp, u32, u64, u32, flt, cint, cint, u32, u32, vp]
    L.elx_put_hypers.restype = cint
    L.elx_put_hypers.argtypes = [vp, u32, vp, vp]
    L.elx_grad_stats_mt_static.restype = cint
    L.elx_grad_stats_mt_static.argtypes = [vp, u32, cint, u32, vp, cint, vp]
    L.elx_adam_step_mt.restype = cint
    L.elx_adam_step_mt.argtypes = [vp, u32, vp, u32, vp, u32, u64, u32, flt, cint, cint, u32, u32, vp]
    L.elx_decide.restype = cint
    L.elx_decide.argtypes = [vp, u32, ctypes.c_double, ctypes.c_double, cint, vp, u32, vp, vp]
    L.elx_adam_step_gated_mt.restype = cint
    L.elx_adam_step_gated_mt.argtypes = [vp, u32, vp, u32, vp, u32, u64, u32, cint, cint, u32, u32, vp]
    L.elx_writeback_mt.restype = cint
    L.elx_writeback_mt.argtypes = [vp, u32, cint, u32, u32, vp]
    L.elx_writeback.restype = cint
    L.elx_writeback.argtypes = [vp, vp, cint, u64, vp]
    L.elx_grad_stats.restype = cint
    L.elx_grad_stats.argtypes = [vp, cint, u64, u32, vp, vp, vp]
    L.elx_land_grads_mt.restype = cint
    L.elx_land_grads_mt.argtypes = [vp, u32, vp, u32, cint, cint, flt, u32, vp, vp, u32, vp]

    if L.elx_version() != ELX_ABI_VERSION:
        raise RuntimeError(f'{LIB_PATH}: ABI version {L.elx_version()} != binding version {ELX_ABI_VERSION}; rebuild')
    built, now = (L.elx_source_sha() or b'').decode(), source_sha16()
    if built != now:
        raise RuntimeError(f'{LIB_PATH} was built from other sources (digest {built or "none"}) than the ones beside it '
                           f'({now}): rebuild with `python -m elixir_amd.build`')
    for name, dt in (('chunk', CHUNK_DTYPE), ('seg', SEG_DTYPE), ('hyper', HYPER_DTYPE), ('stats', STATS_DTYPE),
                     ('decision', DECISION_DTYPE), ('step_ctl', STEP_CTL_DTYPE), ('step_report', STEP_REPORT_DTYPE)):
        size = getattr(L, f'elx_sizeof_{name}')()
        if size != dt.itemsize:
            raise RuntimeError(f'{LIB_PATH}: sizeof {name} record is {size}, binding expects {dt.itemsize}')
    _lib = L
    return L


def _bind_host(L) -> None:
    """Signatures of the entry points that the host-only source file defines."""
    u32, u64, vp, cint, flt = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.elx_check_tables.restype = cint
    L.elx_check_tables.argtypes = [vp, u32, vp, u32, u32, cint, cint, ctypes.POINTER(u64), ctypes.POINTER(u32),
                                   ctypes.POINTER(cint)]
    L.elx_check_land_rows.restype = cint
    L.elx_check_land_rows.argtypes = [vp, u32, vp, u32, cint, cint, ctypes.POINTER(u32)]
    L.elx_land_tile_elems.restype = u32
    L.elx_land_tile_elems.argtypes = [cint]
    for name in ('elx_tile_elems', 'elx_land_max_blocks'):
        getattr(L, name).restype = u32
        getattr(L, name).argtypes = []
    L.elx_unscale_mode.restype = cint
    L.elx_unscale_mode.argtypes = [flt, ctypes.POINTER(flt)]
    L.elx_occupancy_lds_bytes.restype = cint
    L.elx_occupancy_lds_bytes.argtypes = [u32, ctypes.POINTER(u32)]


_host_lib = None


def host_lib() -> ctypes.CDLL:
    """The library whose validators (and other host-only entry points) are called: ``libelx_hip.so``, or --
    for the test run that puts the validators under AddressSanitizer / UBSan -- the build of the host-only
    source file that the environment variable ELX_HOST_CHECKED_LIB names."""
    global _host_lib
    path = os.environ.get('ELX_HOST_CHECKED_LIB')
    if not path:
        return load()
    if _host_lib is None:
        L = ctypes.CDLL(path)
        _bind_host(L)
        _host_lib = L
    return _host_lib


def unscale_mode(div_scale: float):
    """(mode, inv_scale): how an update launch divides by ``div_scale`` (0 not at all, 1 exact multiply, 2 division)."""
    inv = ctypes.c_float(0.0)
    mode = host_lib().elx_unscale_mode(div_scale, ctypes.byref(inv))
    return int(mode), float(inv.value)


def occupancy_lds_bytes(blocks_per_cu: int) -> int:
    lds = ctypes.c_uint32(0)
    code = host_lib().elx_occupancy_lds_bytes(blocks_per_cu, ctypes.byref(lds))
    if code != 0:
        raise ElxError('elx_occupancy_lds_bytes', code, load().elx_strerror(code).decode())
    return int(lds.value)


def check(func: str, code: int) -> None:
    if code != 0:
        raise ElxError(func, code, load().elx_strerror(code).decode())


def tile_elems() -> int:
    return int(host_lib().elx_tile_elems())


def _np_ptr(a: Optional[np.ndarray]):
    if a is None or a.size == 0:
        return None
    assert a.flags['C_CONTIGUOUS']
    return a.ctypes.data_as(ctypes.c_void_p)


class TableInfo(tuple):
    """(total_tiles, max_tiles_per_chunk, all_aligned16) as reported by elx_check_tables, optionally followed
    by the caller's choice of cache policy for the update launch: 0 every access streams, 1 the low-precision
    copy is stored through the memory-side cache (``ELX_FLAG_KEEP_CACHED``), 2 the whole state of the launch
    fits that cache and stays there (``ELX_FLAG_KEEP_STATE_CACHED``)."""
    __slots__ = ()

    @property
    def total_tiles(self) -> int:
        return self[0]

    @property
    def max_tiles(self) -> int:
        return self[1]

    @property
    def aligned(self) -> bool:
        return self[2]

    @property
    def cache_policy(self) -> int:
        return int(self[3]) if len(self) > 3 else 0

    @property
    def keep_lowp_cached(self) -> bool:
        return self.cache_policy >= 1

    @property
    def keep_state_cached(self) -> bool:
        return self.cache_policy >= 2

    def with_cache_policy(self, policy: int) -> 'TableInfo':
        assert policy in (0, 1, 2)
        return TableInfo(tuple(self[:3]) + (int(policy), ))

    def with_keep_lowp_cached(self, keep: bool) -> 'TableInfo':
        return self.with_cache_policy(1 if keep else 0)

    @property
    def flags(self) -> int:
        """The ``flags`` argument of the update launches for these tables."""
        return ((0 if self[2] else ELX_FLAG_SCALAR_ONLY) | (ELX_FLAG_KEEP_CACHED if self.cache_policy >= 1 else 0)
                | (ELX_FLAG_KEEP_STATE_CACHED if self.cache_policy >= 2 else 0))


def check_tables(chunks: np.ndarray, segs: Optional[np.ndarray], n_hypers: int, grad_dtype: int,
                 lowp_dtype: int) -> TableInfo:
    """Validate host tables; returns (total_tiles, max_tiles_per_chunk, all_aligned16)."""
    assert chunks.dtype == CHUNK_DTYPE
    n_segs = 0 if segs is None else len(segs)
    if n_segs:
        assert segs.dtype == SEG_DTYPE
    tiles = ctypes.c_uint64(0)
    max_tiles = ctypes.c_uint32(0)
    aligned = ctypes.c_int(0)
    code = host_lib().elx_check_tables(_np_ptr(chunks), len(chunks), _np_ptr(segs), n_segs, n_hypers, grad_dtype, lowp_dtype,
                                   ctypes.byref(tiles), ctypes.byref(max_tiles), ctypes.byref(aligned))
    check('elx_check_tables', code)
    return TableInfo((int(tiles.value), int(max_tiles.value), bool(aligned.value)))


def stats_flags(scalar_only: bool, keep_cached: bool) -> int:
    return (ELX_FLAG_SCALAR_ONLY if scalar_only else 0) | (ELX_FLAG_KEEP_CACHED if keep_cached else 0)


def grad_stats_mt(d_chunks: int, n_chunks: int, grad_dtype: int, blocks_per_chunk: int, d_partials: int, d_stats: int,
                  scalar_only: bool, stream: int, keep_cached: bool = False) -> None:
    """``keep_cached``: ordinary instead of non-temporal loads, for a gradient set that fits the
    memory-side cache and is read again by the update launch right behind."""
    check('elx_grad_stats_mt',
          load().elx_grad_stats_mt(d_chunks, n_chunks, grad_dtype, blocks_per_chunk, d_partials, d_stats,
                                   stats_flags(scalar_only, keep_cached), stream))


def grad_partials_mt(d_chunks: int, n_chunks: int, grad_dtype: int, blocks_per_chunk: int, d_partials: int,
                     scalar_only: bool, stream: int, keep_cached: bool = False) -> None:
    """The first launch of ``grad_stats_mt`` alone: the partials are left for ``finish_decide``."""
    check('elx_grad_partials_mt',
          load().elx_grad_partials_mt(d_chunks, n_chunks, grad_dtype, blocks_per_chunk, d_partials,
                                      stats_flags(scalar_only, keep_cached), stream))


def finish_decide(d_partials: int, n_chunks: int, blocks_per_chunk: int, d_stats: int, ctl: int, d_hypers: int,
                  max_hypers: int, d_decision: int, report: int, d_counter: int, stream: int, d_rows: int = 0,
                  d_gated_rows: int = 0, n_rows: int = 0, d_armed: int = 0) -> None:
    """Fold of the partials + the decisions of the step, everything that changes read from ``ctl``.  With
    ``d_gated_rows`` (a second device copy of the ``n_rows`` update rows at ``d_rows``, the table of the gated
    update launch that follows) the launch also keeps that table's n_valid column: zeros when the step is
    skipped, the counts of ``d_rows`` again at the first step that happens afterwards (``d_armed``: one
    uint32 of device memory that says which of the two the table holds; 0 for a fresh copy)."""
    if d_gated_rows:
        check('elx_finish_decide_rows',
              load().elx_finish_decide_rows(d_partials, n_chunks, blocks_per_chunk, d_stats, ctl, d_hypers, max_hypers,
                                            d_decision, report or None, d_counter, d_rows, d_gated_rows, n_rows, d_armed, stream))
        return
    check('elx_finish_decide',
          load().elx_finish_decide(d_partials, n_chunks, blocks_per_chunk, d_stats, ctl, d_hypers, max_hypers, d_decision,
                                   report or None, d_counter, stream))


def put_hypers(hyper_host: np.ndarray, d_hypers: int, stream: int) -> None:
    """Host hyper records -> device table, through the arguments of a tiny launch on ``stream``."""
    assert hyper_host.dtype == HYPER_DTYPE
    check('elx_put_hypers', load().elx_put_hypers(_np_ptr(hyper_host), len(hyper_host), d_hypers, stream))


def max_ctl_hypers() -> int:
    return int(load().elx_max_ctl_hypers())


def static_partials() -> int:
    return int(load().elx_static_partials())


def grad_stats_mt_static(d_chunks: int, n_chunks: int, grad_dtype: int, blocks_per_chunk: int, d_stats: int,
                         scalar_only: bool, stream: int, keep_cached: bool = False) -> None:
    """``grad_stats_mt`` with the partials in the library's fixed device array: allocates nothing.  The
    stream's device must be the current one; overlapping calls on one GPU race."""
    check('elx_grad_stats_mt_static',
          load().elx_grad_stats_mt_static(d_chunks, n_chunks, grad_dtype, blocks_per_chunk, d_stats,
                                          stats_flags(scalar_only, keep_cached), stream))


def adam_step_mt(d_chunks: int, n_chunks: int, d_segs: int, n_segs: int, d_hypers: int, n_hypers: int, info: TableInfo,
                 div_scale: float, grad_dtype: int, lowp_dtype: int, blocks_per_cu: int, stream: int) -> None:
    """2-D grid (max tiles per record, records)."""
    check('elx_adam_step_mt',
          load().elx_adam_step_mt(d_chunks, n_chunks, d_segs, n_segs, d_hypers, n_hypers, info.total_tiles,
                                  info.max_tiles, div_scale, grad_dtype, lowp_dtype, info.flags, blocks_per_cu, stream))


def adam_step_put_mt(d_chunks: int, n_chunks: int, d_segs: int, n_segs: int, hyper_host: np.ndarray, d_hypers: int,
                     info: TableInfo, div_scale: float, grad_dtype: int, lowp_dtype: int, blocks_per_cu: int,
                     stream: int) -> None:
    """The update with its hyper records taken from host memory: up to 32 ride in the arguments of the
    update launch itself (``d_hypers`` is then not written), more go through ``put_hypers`` into ``d_hypers``."""
    assert hyper_host.dtype == HYPER_DTYPE
    check('elx_adam_step_put_mt',
          load().elx_adam_step_put_mt(d_chunks, n_chunks, d_segs, n_segs, _np_ptr(hyper_host), d_hypers, len(hyper_host),
                                      info.total_tiles, info.max_tiles, div_scale, grad_dtype, lowp_dtype, info.flags,
                                      blocks_per_cu, stream))


def decide(d_stats: int, n_chunks: int, loss_scale: float, max_norm: float, clipping: bool, d_hypers: int,
           n_hypers: int, d_decision: int, stream: int) -> None:
    check('elx_decide',
          load().elx_decide(d_stats, n_chunks, loss_scale, max_norm, int(clipping), d_hypers, n_hypers, d_decision, stream))


def adam_step_gated_mt(d_chunks: int, n_chunks: int, d_segs: int, n_segs: int, d_hypers: int, n_hypers: int,
                       info: TableInfo, grad_dtype: int, lowp_dtype: int, blocks_per_cu: int, stream: int) -> None:
    """``adam_step_mt`` with the unscale parameters and the skip flag read from the hyper records."""
    check('elx_adam_step_gated_mt',
          load().elx_adam_step_gated_mt(d_chunks, n_chunks, d_segs, n_segs, d_hypers, n_hypers, info.total_tiles,
                                        info.max_tiles, grad_dtype, lowp_dtype, info.flags, blocks_per_cu, stream))


def refresh_piece_elems() -> int:
    return int(load().elx_refresh_piece_elems())


def writeback_mt(d_chunks: int, n_chunks: int, lowp_dtype: int, max_elems: int, aligned: bool, stream: int) -> None:
    """``max_elems``: the largest n_alloc among the records (sizes the grid)."""
    piece = refresh_piece_elems()
    blocks = max(1, min(1 << 20, (max_elems + piece - 1) // piece))    # one piece per workgroup
    check('elx_writeback_mt',
          load().elx_writeback_mt(d_chunks, n_chunks, lowp_dtype, blocks, 0 if aligned else ELX_FLAG_SCALAR_ONLY, stream))


def land_max_blocks() -> int:
    return int(load().elx_land_max_blocks())


def land_tile_elems(src_dtype: int) -> int:
    return int(host_lib().elx_land_tile_elems(src_dtype))


def land_fold_blocks() -> int:
    return int(load().elx_land_fold_blocks())


def land_workspace_records(n_rows: int, blocks_per_row: int, n_slots: int = 0) -> int:
    """ElxStats records the landing launch needs as workspace."""
    return n_rows * blocks_per_row + (n_slots or n_rows) * land_fold_blocks()


def land_grads_mt(d_rows: int, n_rows: int, src_dtype: int, dst_dtype: int, mul: float, blocks_per_row: int,
                  d_partials: int, d_stats: int, aligned: bool, stream: int, blocks_per_cu: int = 0,
                  d_slot_offsets: int = 0, n_slots: int = 0, keep_cached: bool = False) -> None:
    """``keep_cached``: ordinary instead of non-temporal stores, for a destination that fits the
    memory-side cache and is read by the optimizer step soon after."""
    flags = stats_flags(not aligned, keep_cached) | ((blocks_per_cu & 0xFF) << 8)
    check('elx_land_grads_mt',
          load().elx_land_grads_mt(d_rows, n_rows, d_slot_offsets or None, n_slots, src_dtype, dst_dtype, mul,
                                   blocks_per_row, d_partials, d_stats, flags, stream))


def check_land_rows(rows: np.ndarray, slot_offsets: Optional[np.ndarray], src_dtype: int, dst_dtype: int) -> int:
    """Validate a host landing table; returns the one-tile-per-workgroup grid width."""
    assert rows.dtype == CHUNK_DTYPE
    n_slots = 0
    if slot_offsets is not None:
        assert slot_offsets.dtype == np.uint32
        n_slots = len(slot_offsets) - 1
    bpr = ctypes.c_uint32(0)
    check('elx_check_land_rows',
          host_lib().elx_check_land_rows(_np_ptr(rows), len(rows), _np_ptr(slot_offsets), n_slots, src_dtype, dst_dtype,
                                     ctypes.byref(bpr)))
    return int(bpr.value)


def writeback(master: int, lowp: int, lowp_dtype: int, n: int, stream: int) -> None:
    """One buffer: lowp[0, n) = cast(master[0, n))."""
    check('elx_writeback', load().elx_writeback(master, lowp, lowp_dtype, n, stream))


def grad_stats(grad: int, grad_dtype: int, n: int, blocks: int, d_partials: int, d_stats: int, stream: int) -> None:
    """One buffer: overflow flag and sum of squares of grad[0, n)."""
    check('elx_grad_stats', load().elx_grad_stats(grad, grad_dtype, n, blocks, d_partials, d_stats, stream))
