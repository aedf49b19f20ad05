"""The C-ABI library without a GPU: it loads, exports every symbol include/elx_abi.h declares, its
record layouts match the Python mirrors, and its host-side table validation returns the documented
codes.  No kernel is launched here."""
import os
import re

import numpy as np
import pytest

from elixir_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'elx_abi.h')


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(elx_[a-z0-9_]+)\s*\(', text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _abi.load()
    names = declared_functions()
    assert names, 'no declarations found in the header'
    for name in names:
        assert hasattr(lib, name), f'{name} is declared in elx_abi.h but not exported'
    assert sorted(_abi.EXPORTS) == names, 'the binding and the header disagree on the entry points'
    assert lib.elx_version() == _abi.ELX_ABI_VERSION


def test_library_carries_the_digest_of_its_sources_and_a_stale_one_is_refused(monkeypatch, tmp_path):
    """An edited kernel must never be measured through an old binary: the build compiles the digest of the
    sources in, the binding compares it with the sources beside it when it loads the library, and the
    test / benchmark entry (``ensure_built``) rebuilds a library that does not match."""
    from elixir_amd import build as B
    lib = _abi.load()
    now = _abi.source_sha16()
    assert len(now) == 16 and lib.elx_source_sha().decode() == now == _abi.built_source_sha(_abi.LIB_PATH)
    assert not B.is_stale()
    assert [os.path.basename(f) for f in _abi.source_files()] == ['elx_host.cpp', 'elx_host.h', 'elx_kernels.hip', 'elx_abi.h']
    # the same library next to sources that have changed since
    monkeypatch.setattr(_abi, '_lib', None)
    monkeypatch.setattr(_abi, 'source_sha16', lambda: '0123456789abcdef')
    with pytest.raises(RuntimeError, match='built from other sources'):
        _abi.load()
    monkeypatch.setattr(B, 'source_sha16', lambda: '0123456789abcdef')
    assert B.is_stale()
    built = []
    monkeypatch.setattr(B, 'build', lambda verbose=False: built.append(1))
    B.ensure_built()
    assert built == [1]
    monkeypatch.undo()
    assert _abi.load().elx_version() == _abi.ELX_ABI_VERSION
    assert _abi.built_source_sha(str(tmp_path / 'missing.so')) == ''


def test_record_layouts_match_the_header():
    lib = _abi.load()
    assert lib.elx_sizeof_chunk() == _abi.CHUNK_DTYPE.itemsize == 72
    assert lib.elx_sizeof_seg() == _abi.SEG_DTYPE.itemsize == 24
    assert lib.elx_sizeof_hyper() == _abi.HYPER_DTYPE.itemsize == 48
    assert lib.elx_sizeof_stats() == _abi.STATS_DTYPE.itemsize == 16
    # field offsets as the C struct lays them out
    assert [_abi.CHUNK_DTYPE.fields[f][1] for f in ('grad', 'lowp_out', 'master', 'm', 'v', 'n_alloc', 'n_valid',
                                                    'tile_begin', 'seg_begin', 'seg_end')] == [0, 8, 16, 24, 32, 40, 48,
                                                                                              56, 64, 68]
    assert [_abi.HYPER_DTYPE.fields[f][1] for f in ('decay_mul', 'l2_wd', 'lerp_w', 'beta2', 'omb2', 'bc2_sqrt', 'eps',
                                                    'neg_step', 'flags')] == [0, 4, 8, 12, 16, 20, 24, 28, 32]
    assert _abi.tile_elems() in (256, 512)


def test_strerror_covers_every_code():
    lib = _abi.load()
    seen = set()
    for code in range(0, -9, -1):
        text = lib.elx_strerror(code).decode()
        assert text and text not in seen
        seen.add(text)
    assert 'unknown' in lib.elx_strerror(-99).decode()


def _row(n=8192, base=0x10000000):
    row = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
    row['grad'] = base
    row['master'] = base + (1 << 20)
    row['m'] = base + (2 << 20)
    row['v'] = base + (3 << 20)
    row['n_alloc'] = n
    row['n_valid'] = n
    row['seg_end'] = 1
    return row


def test_check_tables_accepts_and_rejects():
    tile = _abi.tile_elems()
    row = _row()
    seg = np.zeros(1, dtype=_abi.SEG_DTYPE)
    seg[0] = (0, 8192, 0, 0)
    info = _abi.check_tables(row, seg, 1, _abi.ELX_F32, _abi.ELX_NONE)
    assert info == (8192 // tile, 8192 // tile, True)

    def expect(code, chunk=row, segs=seg, n_hypers=1, gd=_abi.ELX_F32, ld=_abi.ELX_NONE):
        with pytest.raises(_abi.ElxError) as e:
            _abi.check_tables(chunk, segs, n_hypers, gd, ld)
        assert e.value.code == code, e.value

    bad = row.copy(); bad['master'] = 0; expect(-1, chunk=bad)                        # NULL
    expect(-2, gd=7)                                                                  # dtype
    expect(-2, gd=_abi.ELX_F16, ld=_abi.ELX_BF16)
    bad = row.copy(); bad['lowp_out'] = 0x20000000; expect(-2, chunk=bad)             # lowp_out without a dtype
    bad = row.copy(); bad['m'] = int(row['m'][0]) + 2; expect(-3, chunk=bad)          # fp32 pointer at +2
    bad = row.copy(); bad['grad'] = int(row['grad'][0]) + 1; expect(-3, chunk=bad, gd=_abi.ELX_F16)
    bad = row.copy(); bad['n_valid'] = 9000; expect(-4, chunk=bad)                    # n_valid > n_alloc
    s2 = seg.copy(); s2[0] = (0, 9000, 0, 0); expect(-4, segs=s2)                     # end > n_valid
    s2 = seg.copy(); s2[0] = (10, 10, 0, 0); expect(-4, segs=s2)                      # empty segment
    s2 = seg.copy(); s2[0] = (0, 8192, 3, 0); expect(-4, segs=s2)                     # hyper index
    bad = row.copy(); bad['n_valid'] = 4096; expect(-4, chunk=bad)                    # segment beyond valid head
    two = np.zeros(2, dtype=_abi.SEG_DTYPE); two[0] = (100, 200, 0, 0); two[1] = (150, 300, 0, 0)
    bad = row.copy(); bad['seg_end'] = 2; expect(-5, chunk=bad, segs=two)             # overlap
    two[0] = (300, 400, 0, 0); two[1] = (100, 200, 0, 0); expect(-5, chunk=bad, segs=two)    # unsorted
    bad = row.copy(); bad['tile_begin'] = 1; expect(-6, chunk=bad)                    # tile bookkeeping
    bad = row.copy(); bad['n_alloc'] = 0; bad['n_valid'] = 0; expect(-7, chunk=bad, segs=None)


def test_check_tables_reports_alignment_and_tile_counts():
    tile = _abi.tile_elems()
    per = 8192 // tile
    rows = np.concatenate([_row(8192, 0x10000000), _row(8192, 0x20000000), _row(5000, 0x30000000)])
    rows['seg_begin'] = 0
    rows['seg_end'] = 0
    rows['tile_begin'] = [0, per, 2 * per]
    info = _abi.check_tables(rows, None, 0, _abi.ELX_F16, _abi.ELX_NONE)
    assert info.total_tiles == 2 * per + (5000 + tile - 1) // tile and info.max_tiles == per and info.aligned
    info = _abi.check_tables(rows[2:], None, 0, _abi.ELX_F16, _abi.ELX_NONE) if False else info
    rows[1]['grad'] += 2    # 2-byte aligned only: legal for fp16, but not vectorisable
    info = _abi.check_tables(rows[:2], None, 0, _abi.ELX_F16, _abi.ELX_NONE)
    assert info.total_tiles == 2 * per and not info.aligned and info.flags == _abi.ELX_FLAG_SCALAR_ONLY


def test_launch_entry_points_reject_bad_arguments_before_launching():
    """Argument errors are returned before any kernel is enqueued, so this runs without a GPU."""
    lib = _abi.load()
    assert lib.elx_grad_stats_mt(None, 1, _abi.ELX_F16, 1, None, None, 0, None) == -1
    assert lib.elx_grad_stats_mt(1, 1, _abi.ELX_F16, 0, 1, 1, 0, None) == -7
    assert lib.elx_grad_stats_mt(1, 1, _abi.ELX_F16, 2000, 1, 1, 0, None) == -7
    assert lib.elx_adam_step_mt(None, 1, None, 0, None, 0, 1, 0, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None) == -1
    assert lib.elx_adam_step_mt(1, 1, None, 0, None, 0, 0, 0, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None) == -7
    assert lib.elx_adam_step_mt(1, 1, None, 0, None, 0, 4, 4, -1.0, 9, _abi.ELX_NONE, 0, 0, None) == -2
    assert lib.elx_adam_step_mt(1, 1, None, 0, None, 0, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 2, None) == -7
    assert lib.elx_adam_step_mt(1, 2, None, 0, None, 0, 5, 2, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None) == -6
    # a grid of zero tiles per record is refused, by both update entry points
    assert lib.elx_adam_step_mt(1, 1, None, 0, None, 0, 4, 0, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None) == -6
    assert lib.elx_adam_step_gated_mt(1, 1, None, 0, None, 0, 4, 0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None) == -6
    # flags of the update launches: scalar-only (1), the two cache policies (2, 4) and their sums; other bits are refused
    assert lib.elx_adam_step_mt(1, 1, None, 0, None, 0, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 8, 0, None) == -4
    assert lib.elx_adam_step_gated_mt(1, 1, None, 0, None, 0, 4, 4, _abi.ELX_F16, _abi.ELX_F16, 16, 0, None) == -4
    assert lib.elx_adam_step_put_mt(8, 1, None, 0, 8, 8, 1, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0x100, 0, None) == -4
    assert _abi.ELX_FLAG_KEEP_STATE_CACHED == 4
    assert lib.elx_writeback_mt(None, 1, _abi.ELX_F16, 4, 0, None) == -1
    assert lib.elx_writeback_mt(1, 1, _abi.ELX_NONE, 4, 0, None) == -2
    assert lib.elx_writeback_mt(1, 1, _abi.ELX_F16, 0, 0, None) == -7
    assert lib.elx_refresh_piece_elems() == 1024
    # the stats launch alone, the fold-and-decide launch, the hyper records through launch arguments
    assert lib.elx_grad_partials_mt(None, 1, _abi.ELX_F16, 1, 1, 0, None) == -1
    assert lib.elx_grad_partials_mt(1, 1, _abi.ELX_F16, 1025, 1, 0, None) == -7
    assert lib.elx_grad_partials_mt(1, 1, 9, 1, 1, 0, None) == -2
    # flags of the stats launches: scalar-only (1), keep-cached (2) or both; anything else is refused
    assert lib.elx_grad_partials_mt(1, 1, _abi.ELX_F16, 1, 1, 4, None) == -4
    assert lib.elx_grad_stats_mt(1, 1, _abi.ELX_F16, 1, 1, 1, 8, None) == -4
    assert lib.elx_grad_stats_mt_static(8, 1, _abi.ELX_F16, 1, 8, 4, None) == -4
    assert _abi.stats_flags(True, True) == 3 and _abi.stats_flags(False, True) == _abi.ELX_FLAG_KEEP_CACHED == 2
    assert lib.elx_max_ctl_hypers() == 256
    assert lib.elx_finish_decide(None, 1, 1, 8, 8, 8, 1, 8, None, 8, None) == -1
    assert lib.elx_finish_decide(8, 1, 1, 8, None, 8, 1, 8, None, 8, None) == -1            # no control block
    assert lib.elx_finish_decide(8, 1, 1, 8, 8, 8, 1, 8, None, None, None) == -1            # no counter
    assert lib.elx_finish_decide(8, 0, 1, 8, 8, 8, 1, 8, None, 8, None) == -7
    assert lib.elx_finish_decide(8, 1, 0, 8, 8, 8, 1, 8, None, 8, None) == -7
    assert lib.elx_finish_decide(8, 1, 1, 8, 8, 8, 257, 8, None, 8, None) == -7            # more records than the block can carry
    assert lib.elx_finish_decide(8, 1, 1, 8, 12, 8, 1, 8, None, 8, None) == -3             # control block not 8-byte aligned
    # the variant that arms a row table: both tables or none, distinct, a sane row count
    rows_args = (8, 1, 1, 8, 8, 8, 1, 8, None, 8)
    assert lib.elx_finish_decide_rows(*rows_args, None, 16, 4, 8, None) == -1       # a table to arm, none to read the counts from
    assert lib.elx_finish_decide_rows(*rows_args, 8, 16, 4, None, None) == -1       # no word that says what the table holds
    assert lib.elx_finish_decide_rows(*rows_args, 16, 16, 4, 8, None) == -4         # one table for both
    assert lib.elx_finish_decide_rows(*rows_args, 8, 16, 0, 8, None) == -7
    assert lib.elx_finish_decide_rows(*rows_args, 8, 16, 70000, 8, None) == -7
    assert lib.elx_finish_decide_rows(*rows_args, 8, 12, 4, 8, None) == -3
    assert lib.elx_finish_decide_rows(*rows_args, 8, 16, 4, 6, None) == -3
    assert lib.elx_finish_decide_rows(None, 1, 1, 8, 8, 8, 1, 8, None, 8, 8, 16, 4, 8, None) == -1
    assert lib.elx_put_hypers(None, 1, 8, None) == -1
    assert lib.elx_put_hypers(8, 0, 8, None) == -7
    assert lib.elx_put_hypers(8, 1, 6, None) == -3
    for args, code in (((8, 1, None, 0, None, 8, 1, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None), -1),
                       ((8, 1, None, 0, 8, 8, 0, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None), -7),
                       ((8, 1, None, 0, 8, 8, 1, 4, 0, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 0, None), -6),
                       ((8, 1, None, 0, 8, 8, 1, 4, 4, -1.0, 9, _abi.ELX_NONE, 0, 0, None), -2),
                       ((8, 1, None, 0, 8, 8, 1, 4, 4, -1.0, _abi.ELX_F16, _abi.ELX_F16, 0, 2, None), -7)):
        assert lib.elx_adam_step_put_mt(*args) == code, args    # refused before the records are even read
    # the variant without a workspace refuses what its fixed array cannot hold, before it looks anything up
    assert lib.elx_static_partials() == 65536
    assert lib.elx_grad_stats_mt_static(8, 65, _abi.ELX_F16, 1024, 8, 0, None) == -7
    assert lib.elx_grad_stats_mt_static(8, 1, 9, 1, 8, 0, None) == -2
    assert lib.elx_grad_stats_mt_static(None, 1, _abi.ELX_F16, 1, 8, 0, None) == -1


def test_check_land_rows_accepts_and_rejects():
    tile = _abi.land_tile_elems(_abi.ELX_F16)
    assert tile == 2048 and _abi.land_tile_elems(_abi.ELX_F32) == 1024
    rows = np.zeros(3, dtype=_abi.CHUNK_DTYPE)
    rows['grad'] = [0x10000000, 0, 0x30000000]
    rows['lowp_out'] = [0x40000000, 0x50000000, 0x60000002]
    rows['n_alloc'] = [5 * tile, 7, 3 * tile + 1]
    rows['n_valid'] = [5 * tile, 0, 3 * tile + 1]
    assert _abi.check_land_rows(rows, None, _abi.ELX_F16, _abi.ELX_F16) == 5
    assert _abi.check_land_rows(rows, np.array([0, 2, 3], dtype=np.uint32), _abi.ELX_F16, _abi.ELX_F16) == 5
    assert _abi.check_land_rows(rows, None, _abi.ELX_F32, _abi.ELX_F16) == 10
    # a row with more tiles than a launch may have workgroups per row: the width is capped, the workgroups stride
    long = rows.copy()
    long['n_alloc'][0] = long['n_valid'][0] = (1 << 32) + 77
    cap = _abi.host_lib().elx_land_max_blocks()
    assert cap == 1 << 20 and _abi.check_land_rows(long, None, _abi.ELX_F16, _abi.ELX_F16) == cap
    long['n_alloc'][0] = long['n_valid'][0] = cap * tile
    assert _abi.check_land_rows(long, None, _abi.ELX_F16, _abi.ELX_F16) == cap
    long['n_alloc'][0] = long['n_valid'][0] = cap * tile - 1
    assert _abi.check_land_rows(long, None, _abi.ELX_F16, _abi.ELX_F16) == cap
    long['n_alloc'][0] = long['n_valid'][0] = (cap - 1) * tile
    assert _abi.check_land_rows(long, None, _abi.ELX_F16, _abi.ELX_F16) == cap - 1

    def expect(code, r=rows, offsets=None, sd=_abi.ELX_F16, dd=_abi.ELX_F16):
        with pytest.raises(_abi.ElxError) as e:
            _abi.check_land_rows(r, offsets, sd, dd)
        assert e.value.code == code, e.value

    expect(_abi.ELX_E_DTYPE, sd=_abi.ELX_F16, dd=_abi.ELX_F32)
    expect(_abi.ELX_E_DTYPE, sd=_abi.ELX_BF16, dd=_abi.ELX_F16)
    bad = rows.copy(); bad['lowp_out'][1] = 0
    expect(_abi.ELX_E_NULL, bad)
    bad = rows.copy(); bad['n_alloc'][0] = 0; bad['n_valid'][0] = 0
    expect(_abi.ELX_E_SIZE, bad)
    bad = rows.copy(); bad['n_valid'][1] = 8
    expect(_abi.ELX_E_RANGE, bad)
    bad = rows.copy(); bad['grad'][0] += 1
    expect(_abi.ELX_E_ALIGN, bad)
    expect(_abi.ELX_E_ALIGN, sd=_abi.ELX_F32, dd=_abi.ELX_F32)            # 0x60000002 is not 4-byte aligned
    expect(_abi.ELX_E_RANGE, offsets=np.array([1, 2, 3], dtype=np.uint32))
    expect(_abi.ELX_E_RANGE, offsets=np.array([0, 2, 2], dtype=np.uint32))
    expect(_abi.ELX_E_ORDER, offsets=np.array([0, 3, 2, 3], dtype=np.uint32))
    expect(_abi.ELX_E_SIZE, offsets=np.array([0, 1, 2, 3, 3], dtype=np.uint32))


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 on its own, and the record sizes a C
    compiler sees must be the ones the library and the binding use."""
    import subprocess
    src = tmp_path / 'probe.c'
    src.write_text('#include "elx_abi.h"\n#include <stdio.h>\n'
                   'int main(void) { printf("%zu %zu %zu %zu %zu\\n", sizeof(ElxChunk), sizeof(ElxSeg), sizeof(ElxHyper), '
                   'sizeof(ElxStats), sizeof(ElxDecision)); return 0; }\n')
    exe = tmp_path / 'probe'
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'include')
    subprocess.run(['gcc', '-std=c99', '-Wall', '-Wextra', '-pedantic', '-Werror', '-I', inc, str(src), '-o', str(exe)],
                   check=True)
    sizes = [int(x) for x in subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout.split()]
    lib = _abi.load()
    assert sizes == [lib.elx_sizeof_chunk(), lib.elx_sizeof_seg(), lib.elx_sizeof_hyper(), lib.elx_sizeof_stats(),
                     lib.elx_sizeof_decision()] == [72, 24, 48, 16, 32]
    assert _abi.DECISION_DTYPE.itemsize == 32


def test_check_tables_property_random():
    """The validator is what stands between a table and a launch.  Whatever table is drawn: if it is
    accepted, every bound the kernels rely on holds (recomputed here); and each single corruption of an
    accepted table is refused with a negative code, never accepted and never a crash."""
    from hypothesis import given, settings, strategies as st
    tile = _abi.tile_elems()

    @st.composite
    def tables(draw):
        n_rows = draw(st.integers(1, 5))
        n_hypers = draw(st.integers(1, 3))
        rows = np.zeros(n_rows, dtype=_abi.CHUNK_DTYPE)
        segs = []
        tiles = 0
        for i in range(n_rows):
            n_alloc = draw(st.integers(1, 50_000))
            n_valid = draw(st.integers(0, n_alloc))
            base = (i + 1) << 32
            rows[i]['grad'] = base if draw(st.booleans()) else 0
            rows[i]['lowp_out'] = base + (1 << 28)
            rows[i]['master'], rows[i]['m'], rows[i]['v'] = base + (2 << 28), base + (3 << 28), base + (4 << 28)
            rows[i]['n_alloc'], rows[i]['n_valid'], rows[i]['tile_begin'] = n_alloc, n_valid, tiles
            tiles += (n_alloc + tile - 1) // tile
            rows[i]['seg_begin'] = len(segs)
            cuts = sorted(set(draw(st.lists(st.integers(0, n_valid), max_size=6)) + [0, n_valid]))
            for a, b in zip(cuts, cuts[1:]):
                if b > a and draw(st.booleans()):
                    segs.append((draw(st.integers(a, b - 1)), b, draw(st.integers(0, n_hypers - 1)), 0))
            rows[i]['seg_end'] = len(segs)
        seg_arr = np.array(segs, dtype=_abi.SEG_DTYPE) if segs else np.zeros(0, dtype=_abi.SEG_DTYPE)
        return rows, seg_arr, n_hypers, tiles

    def refused(rows, segs, n_hypers, gd=_abi.ELX_F16, ld=_abi.ELX_F16):
        try:
            _abi.check_tables(rows, segs if len(segs) else None, n_hypers, gd, ld)
        except _abi.ElxError as e:
            assert e.code < 0
            return True
        return False

    @settings(max_examples=150, deadline=None, derandomize=True, database=None)
    @given(tables(), st.randoms(use_true_random=False))
    def run(table, rnd):
        rows, segs, n_hypers, tiles = table
        info = _abi.check_tables(rows, segs if len(segs) else None, n_hypers, _abi.ELX_F16, _abi.ELX_F16)
        assert info.total_tiles == tiles and info.aligned
        assert info.max_tiles == max((int(r['n_alloc']) + tile - 1) // tile for r in rows)
        i = rnd.randrange(len(rows))
        corruptions = [
            lambda r, s: r[i].__setitem__('master', 0),
            lambda r, s: r[i].__setitem__('m', int(r[i]['m']) + 1),
            lambda r, s: r[i].__setitem__('grad', int(r[i]['lowp_out']) + 1),
            lambda r, s: r[i].__setitem__('n_valid', int(r[i]['n_alloc']) + 1),
            lambda r, s: r[i].__setitem__('n_alloc', 0),
            lambda r, s: r[i].__setitem__('n_alloc', (1 << 40) + 1),
            lambda r, s: r[i].__setitem__('tile_begin', int(r[i]['tile_begin']) + 1),
            lambda r, s: r[i].__setitem__('seg_end', len(s) + 1),
            lambda r, s: r[i].__setitem__('seg_begin', int(r[i]['seg_end']) + 1),
        ]
        if len(segs):
            j = rnd.randrange(len(segs))
            owner = next(k for k in range(len(rows)) if rows[k]['seg_begin'] <= j < rows[k]['seg_end'])
            corruptions += [
                lambda r, s: s[j].__setitem__('hyper', n_hypers),
                lambda r, s: s[j].__setitem__('end', int(r[owner]['n_valid']) + 1),
                lambda r, s: s[j].__setitem__('begin', int(s[j]['end'])),
            ]
            if j + 1 < rows[owner]['seg_end']:
                corruptions.append(lambda r, s: s[j].__setitem__('end', int(s[j + 1]['begin']) + 1))
        for corrupt in corruptions:
            r2, s2 = rows.copy(), segs.copy()
            corrupt(r2, s2)
            assert refused(r2, s2, n_hypers), (corruptions.index(corrupt), r2, s2)
        assert refused(rows, segs, n_hypers, gd=_abi.ELX_F16, ld=_abi.ELX_BF16)
        assert refused(rows, segs, n_hypers, gd=5)
        if len(segs):
            assert refused(rows, segs, 0)

    run()


def test_missing_library_and_missing_gpu_fail_loudly(monkeypatch):
    """There is no CPU path behind the optimizer: without the built library every entry raises and
    says how to build it, and parameters that are not on a GPU are refused by name of the reason."""
    import torch
    import elixir_amd as ea
    monkeypatch.setattr(_abi, '_lib', None)
    monkeypatch.setattr(_abi, 'LIB_PATH', os.path.join(ROOT, 'elixir_amd', 'no_such_library.so'))
    with pytest.raises(RuntimeError, match='has not been built'):
        _abi.load()
    with pytest.raises(RuntimeError, match='no CPU fallback'):
        _abi.tile_elems()
    monkeypatch.undo()
    assert _abi.tile_elems() == 256
    p = torch.nn.Parameter(torch.zeros(8))
    p.grad = torch.ones(8)
    with pytest.raises(RuntimeError, match='runs on the GPU'):
        ea.HybridAdam([p]).step()
    assert torch.count_nonzero(p.data) == 0          # nothing was updated by some other route


def test_device_code_has_no_packed_fp32_and_no_spills(tmp_path):
    """What the build flags promise about the device code, checked on the compiler's own listing:
    no packed-fp32 arithmetic (the kernels' fp32 results must not depend on how the compiler pairs
    lanes' operands), no register spills and no private memory in any kernel."""
    import subprocess
    from elixir_amd import build as B
    asm = tmp_path / 'elx.s'
    flags = [f for f in B.HIPCC_FLAGS if f not in ('-shared', '-fPIC')]
    subprocess.run([B.hipcc_path()] + flags + ['--cuda-device-only', '-S', '-I', os.path.join(ROOT, 'include'), '-o', str(asm)]
                   + B.SOURCES[:1], check=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    text = asm.read_text()
    assert not re.search(r'\bv_pk_(add|mul|fma)_f32\b', text)
    kernels = re.findall(r'\.amdhsa_kernel\s+(\S+)', text)
    assert len(kernels) >= 30
    for key in ('.private_segment_fixed_size', '.sgpr_spill_count', '.vgpr_spill_count'):
        values = re.findall(re.escape(key) + r':\s*(\d+)', text)
        assert len(values) == len(kernels) and set(values) == {'0'}, (key, set(values))
    # the update kernels keep a small register footprint: residency is capped by the LDS reservation, not by registers
    vgprs = [int(v) for v in re.findall(r'\.vgpr_count:\s*(\d+)', text)]
    assert max(vgprs) <= 128


def test_unscale_mode_and_lds_reservation_queries():
    """How a launch divides by div_scale, and the LDS reservation that caps residency, as the library's own
    host code decides them: the exact-reciprocal rule against its definition (a power of two whose reciprocal
    is a normal fp32 number), on every power of two and on neighbours of powers of two."""
    assert _abi.unscale_mode(-1.0) == (0, 1.0) and _abi.unscale_mode(0.0) == (0, 1.0)
    assert _abi.unscale_mode(float('nan'))[0] == 0
    for e in range(-149, 128):
        s = float(np.ldexp(np.float32(1.0), e))
        mode, inv = _abi.unscale_mode(s)
        with np.errstate(all='ignore'):
            recip = np.float32(1.0) / np.float32(s)
        # both the divisor and its reciprocal normal numbers; 2**126, whose reciprocal is the smallest normal
        # number, is left to the division (same bits either way)
        exact = -126 <= e <= 125
        assert not exact or (np.isfinite(recip) and recip >= np.float32(1.17549435e-38) and recip * np.float32(s) == 1.0)
        assert mode == (1 if exact else 2), (e, mode)
        assert inv == (float(recip) if exact else 1.0)
        if -126 <= e < 127:
            for neighbour in (np.nextafter(np.float32(s), np.float32(np.inf)), np.nextafter(np.float32(s), np.float32(0))):
                assert _abi.unscale_mode(float(neighbour)) == (2, 1.0)
    assert _abi.unscale_mode(float('inf')) == (2, 1.0)
    # the reservation: a multiple of 256 bytes that lets exactly the asked number of workgroups share 160 KiB
    for k in range(3, 33):
        lds = _abi.occupancy_lds_bytes(k)
        assert lds % 256 == 0 and lds <= 65536 and (160 * 1024) // lds >= k and (160 * 1024) // (lds + 256) <= k
    assert _abi.occupancy_lds_bytes(0) == _abi.occupancy_lds_bytes(12)
    for bad in (1, 2, 33, 1000):
        with pytest.raises(_abi.ElxError) as e:
            _abi.occupancy_lds_bytes(bad)
        assert e.value.code == _abi.ELX_E_SIZE


SANITIZED_TESTS = ('test_check_tables_property_random', 'test_check_tables_accepts_and_rejects',
                   'test_check_tables_reports_alignment_and_tile_counts', 'test_check_land_rows_accepts_and_rejects',
                   'test_unscale_mode_and_lds_reservation_queries')


def test_validators_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """The table validators are what keeps a kernel inside its buffers, so their own reads must stay inside
    the tables they are given: the host-only source file of the library is compiled alone with g++
    -fsanitize=address,undefined, and the validator tests of this file (and the land-row tests of
    test_host_logic.py) run once more against that build, in a child process whose allocator is
    AddressSanitizer's (every numpy table then sits between red zones).  A read or write outside a table, or
    any undefined arithmetic, ends the child with a report."""
    import subprocess
    import sys
    from elixir_amd import build as B
    if os.environ.get('ELX_HOST_CHECKED_LIB'):
        pytest.skip('this is the child run')
    lib = B.build_host_checked(str(tmp_path / 'libelx_host_checked.so'))
    asan = subprocess.run(['g++', '-print-file-name=libasan.so'], check=True, stdout=subprocess.PIPE, text=True).stdout.strip()
    asan = os.path.realpath(asan)
    assert os.path.exists(asan), 'the AddressSanitizer runtime of g++ was not found'
    env = dict(os.environ)
    env['ELX_HOST_CHECKED_LIB'] = lib
    # the runtime has to be the first library of the process; whatever else is preloaded stays behind it
    env['LD_PRELOAD'] = asan + (':' + env['LD_PRELOAD'] if env.get('LD_PRELOAD') else '')
    env['ASAN_OPTIONS'] = 'detect_leaks=0:abort_on_error=0:exitcode=97'
    env['UBSAN_OPTIONS'] = 'halt_on_error=1:print_stacktrace=1'
    here = os.path.dirname(os.path.abspath(__file__))
    select = ' or '.join(SANITIZED_TESTS + ('test_land_rows_tile_every_piece_exactly', 'test_launch_plan_properties_random'))
    proc = subprocess.run([sys.executable, '-m', 'pytest', '-x', '-q', '-p', 'no:cacheprovider',
                           os.path.join(here, 'test_abi.py'), os.path.join(here, 'test_host_logic.py'), '-k', select],
                          env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    tail = proc.stdout[-3000:]
    assert proc.returncode == 0, tail
    assert 'passed' in tail and 'ERROR: AddressSanitizer' not in proc.stdout and 'runtime error' not in proc.stdout, tail
    # and the child really called into the checked build
    probe = subprocess.run([sys.executable, '-c',
                            'import sys; sys.path.insert(0, sys.argv[1]); from elixir_amd import _abi; '
                            'L = _abi.host_lib(); print(L._name); print(_abi.tile_elems())', ROOT],
                           env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert probe.returncode == 0 and 'libelx_host_checked.so' in probe.stdout and '256' in probe.stdout, probe.stdout[-2000:]
