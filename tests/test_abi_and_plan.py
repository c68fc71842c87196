"""CPU-side checks of the shared library: it loads without a GPU, exports every
entry point include/cuvdia.h declares, fails loudly (not silently) when asked
to compute without a device, and its host-only chunk planner decomposes offset
tables correctly."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "cuvdia.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cuvdia_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("cuvdia_spmm_f32", "cuvdia_dd2dia_f32", "cuvdia_desc_create", "cuvdia_desc_destroy",
                 "cuvdia_strerror", "cuvdia_plan_chunks", "cuvdia_spmm_offsets_f32", "cuvdia_dd2dia_offsets_f32"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from cuv_amd import _lib
    L = _lib.lib()
    for name in _declared():
        assert hasattr(L, name), "libcuvdia.so does not export %s" % name
    assert L.cuvdia_abi_version() == 1
    assert L.cuvdia_strerror(-2).decode() == "operand shapes do not match the matrix"
    assert L.cuvdia_strerror(0).decode() == "ok"


def test_no_device_is_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from cuv_amd import _lib
    L = _lib.lib()
    d = ctypes.c_void_p()
    offs = np.array([0, 1], np.int32)
    rc = L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 2, 8, 8, 8, 1)
    assert rc == _lib.ENODEVICE and not d.value
    # argument validation still happens first
    rc = L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 2, 8, 8, 4, 1)
    assert rc == _lib.EINVAL
    assert L.cuvdia_spmm_f32(None, None, None, 0, None, 0, 1, b"n", 1.0, 0.0, None) == _lib.EINVAL
    assert L.cuvdia_set_path(7) == _lib.EINVAL and L.cuvdia_set_path(0) == 0
    # argument checks come before any device work
    assert L.cuvdia_learn_step_weight_decay_f32(None, None, -1, 0.1, 0.0, None) == _lib.EINVAL
    assert L.cuvdia_learn_step_weight_decay_f32(None, None, 0, 0.1, 0.0, None) == 0
    assert L.cuvdia_learn_step_weight_decay_f32(None, None, 4, 0.1, 0.0, None) == _lib.EINVAL
    assert L.cuvdia_learn_step_weight_decay_momentum_f32(None, None, None, -1, 0.1, 0.9, 0.0, None) == _lib.EINVAL
    assert L.cuvdia_learn_step_weight_decay_momentum_f32(None, None, None, 0, 0.1, 0.9, 0.0, None) == 0
    assert L.cuvdia_learn_step_weight_decay_momentum_f32(None, None, None, 4, 0.1, 0.9, 0.0, None) == _lib.EINVAL
    assert L.cuvdia_spmm_layer_f32(None, None, None, 0, None, 0, 1, b"n", 1.0, 0.0, None, 7, 0, None) == _lib.EINVAL
    assert L.cuvdia_spmm_bias_act_f32(None, None, None, 0, None, 0, 1, b"n", 1.0, 0.0, None,
                                      _lib.ACT_SIGMOID_SAMPLE, None) == _lib.EINVAL


def _plan(offsets, transposed=False, max_len=8):
    from cuv_amd import _lib
    L = _lib.lib()
    offs = np.ascontiguousarray(offsets, np.int32)
    ip = ctypes.POINTER(ctypes.c_int)
    if max_len == 8:
        def call(*out):
            return L.cuvdia_plan_chunks(offs.ctypes.data_as(ip), offs.size, int(transposed), *out)
    else:
        def call(*out):
            return L.cuvdia_plan_chunks_max(offs.ctypes.data_as(ip), offs.size, int(transposed), max_len, *out)
    n = call(None, None, None, 0)
    assert n > 0
    s0, ln, sl = np.zeros(n, np.int32), np.zeros(n, np.int32), np.zeros(max_len * n, np.int32)
    assert call(s0.ctypes.data_as(ip), ln.ctypes.data_as(ip), sl.ctypes.data_as(ip), n) == n
    return s0, ln, sl.reshape(n, max_len)


def _check_plan_covers(offsets, transposed, max_len=8):
    s0, ln, sl = _plan(offsets, transposed, max_len)
    sign = -1 if transposed else 1
    seen = []
    for c in range(len(s0)):
        assert 1 <= ln[c] <= max_len
        for j in range(max_len):
            if j < ln[c] and sl[c, j] >= 0:
                assert sign * offsets[sl[c, j]] == s0[c] + j       # the slot really has that shift
                seen.append(int(sl[c, j]))
            else:
                assert sl[c, j] == -1
    assert sorted(seen) == list(range(len(offsets)))             # every diagonal exactly once
    assert all(s0[i] <= s0[i + 1] for i in range(len(s0) - 1))
    return s0, ln, sl


def test_plan_window_pattern():
    offs = [dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    s0, ln, sl = _check_plan_covers(offs, False)
    assert s0.tolist() == [dy * 128 - 3 for dy in range(-3, 4)] and ln.tolist() == [7] * 7
    assert sl[0, :7].tolist() == list(range(7))
    s0t, lnt, slt = _check_plan_covers(offs, True)
    assert s0t.tolist() == [dy * 128 - 3 for dy in range(-3, 4)]
    assert slt[0, :7].tolist() == [48, 47, 46, 45, 44, 43, 42]     # shifts are negated offsets


def test_plan_long_runs_are_split_evenly():
    s0, ln, _ = _check_plan_covers(list(range(-16, 17)), False)     # one run of 33
    assert ln.tolist() == [7, 7, 7, 6, 6] and s0[0] == -16
    offs = [c * 65536 + dy * 256 + dx for c in range(4) for dy in range(-6, 7) for dx in range(-6, 7)]
    s0, ln, _ = _check_plan_covers(offs, False)                     # 52 runs of 13 -> 7 + 6
    assert len(s0) == 104 and sorted(set(ln.tolist())) == [6, 7]


def test_plan_of_the_products_takes_chunks_of_13():
    """The products' tables: a 13-wide window row is one chunk, longer runs are cut evenly."""
    offs = [c * 65536 + dy * 256 + dx for c in range(4) for dy in range(-6, 7) for dx in range(-6, 7)]
    for transposed in (False, True):
        s0, ln, sl = _check_plan_covers(offs, transposed, 13)
        assert len(s0) == 52 and set(ln.tolist()) == {13}
    s0, ln, _ = _check_plan_covers(list(range(-16, 17)), False, 13)      # one run of 33 -> 11 + 11 + 11
    assert ln.tolist() == [11, 11, 11] and s0.tolist() == [-16, -5, 6]
    s0, ln, _ = _check_plan_covers([dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)], False, 13)
    assert ln.tolist() == [7] * 7                                         # runs of 7 stay as they are
    _check_plan_covers([0, 0, 3, 2000, -2000, 3], True, 13)
    _check_plan_covers(list(range(40)), False, 1)


def test_plan_isolated_and_adjacent_runs():
    offs = [0, 1, -1, 10, 11, 12, 13, 14, 15, 16, 17, 18, 40]
    s0, ln, sl = _check_plan_covers(offs, False)
    assert s0.tolist() == [-1, 10, 15, 40] and ln.tolist() == [3, 5, 4, 1]
    assert sl[0, :3].tolist() == [2, 0, 1]
    _check_plan_covers(offs, True)


def test_plan_unsorted_duplicates_and_extremes():
    _check_plan_covers([5, -7, 0, 39, -39], False)
    s0, ln, sl = _check_plan_covers([0, 0, 3, 2000, -2000, 3], False)   # a repeated offset opens a new run
    assert len(s0) >= 5
    _check_plan_covers([7], True)


def test_plan_rejects_bad_arguments():
    from cuv_amd import _lib
    L = _lib.lib()
    assert L.cuvdia_plan_chunks(None, 3, 0, None, None, None, 0) == _lib.EINVAL
    three = np.arange(3, dtype=np.int32).ctypes.data_as(ctypes.POINTER(ctypes.c_int))
    assert L.cuvdia_plan_chunks_max(three, 3, 0, 0, None, None, None, 0) == _lib.EINVAL
    assert L.cuvdia_plan_chunks_max(three, 3, 0, 14, None, None, None, 0) == _lib.EINVAL
    offs = np.array([1], np.int32)
    assert L.cuvdia_plan_chunks(offs.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), 0, 0, None, None, None, 0) == _lib.EINVAL


def _units(offs):
    from cuv_amd import _lib
    L = _lib.lib()
    ip = ctypes.POINTER(ctypes.c_int)
    offs = np.ascontiguousarray(offs, np.int32)
    n = L.cuvdia_plan_units(offs.ctypes.data_as(ip), offs.size, None, None, 0)
    assert n >= 1
    c1, c2 = np.zeros(n, np.int32), np.zeros(n, np.int32)
    assert L.cuvdia_plan_units(offs.ctypes.data_as(ip), offs.size, c1.ctypes.data_as(ip), c2.ctypes.data_as(ip), n) == n
    return list(zip(c1.tolist(), c2.tolist()))


def test_units_pair_window_rows():
    # 7x7 window on a 128-wide map: 7 chunks with first shifts 128 apart -> 3 pairs and a single
    offs = [dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    assert _units(offs) == [(0, 1), (2, 3), (4, 5), (6, -1)]
    # every chunk appears exactly once, in order
    for o in ([0], list(range(-20, 21)), [5, -7, 0, 39, -39], [dy * 64 + dx for dy in range(5) for dx in range(8)]):
        got = _units(o)
        flat = [c for u in got for c in u if c >= 0]
        assert flat == list(range(len(_plan(o, False)[0])))


def test_units_pairing_rule():
    # first shifts a multiple of 4 and at most 4096 apart: a pair; 7 apart, 258 apart or 4100 apart: singles
    assert _units(list(range(-8, -1)) + list(range(0, 8))) == [(0, 1)]
    assert _units(list(range(0, 13))) == [(0, -1), (1, -1)]                 # one run of 13 -> chunks 7 + 6, shifts 7 apart
    assert _units([0, 1, 258, 259]) == [(0, -1), (1, -1)]
    assert _units([0, 1, 260, 261]) == [(0, 1)]
    assert _units([0, 1, 4096, 4097]) == [(0, 1)]
    assert _units([0, 1, 4100, 4101]) == [(0, -1), (1, -1)]
    assert _units([0, 1, 132, 133]) == [(0, 1)]
    assert _units([0, 1, 256, 257, 512]) == [(0, 1), (2, -1)]
    assert _units([0, 1, 128, 129, 256]) == [(0, 1), (2, -1)]
    from cuv_amd import _lib
    assert _lib.lib().cuvdia_plan_units(None, 3, None, None, 0) == _lib.EINVAL


# ------------------------------------------------------------------ file io ---
def test_dia_file_round_trip(tmp_path):
    """The seven fields of sparse_matrix_io.hpp:52-66, same names and order,
    survive a save/load; malformed field sets are rejected with the
    constructor's own conditions (dia_matrix.hpp:98-109,131)."""
    from cuv_amd import io
    rng = np.random.default_rng(5)
    offs = np.array([0, 3, -2, 17], np.int32)
    f = dict(m_width=20, m_height=33, m_num_dia=4, m_stride=33, m_row_fact=1, m_offsets=offs,
             m_vec=rng.normal(size=4 * 33).astype(np.float32))
    path = str(tmp_path / "w.npz")
    io.save_fields(path, f)
    with np.load(path) as z:
        assert tuple(z.files) == io.FIELDS
    g = io.load_fields(path)
    assert tuple(g) == io.FIELDS
    assert [int(g[k]) for k in io.FIELDS[:5]] == [20, 33, 4, 33, 1]
    assert np.array_equal(g["m_offsets"], offs) and g["m_offsets"].dtype == np.int32
    assert np.array_equal(g["m_vec"], f["m_vec"]) and g["m_vec"].dtype == np.float32
    with pytest.raises(RuntimeError):
        io.check_fields(dict(f, m_row_fact=0))
    with pytest.raises(RuntimeError):
        io.check_fields(dict(f, m_stride=19))
    with pytest.raises(ValueError):
        io.check_fields(dict(f, m_vec=f["m_vec"][:-1]))
    with pytest.raises(ValueError):
        io.check_fields({k: v for k, v in f.items() if k != "m_offsets"})


def _walk(offs, stride, transposed=0):
    from cuv_amd import _lib
    L = _lib.lib()
    ip = ctypes.POINTER(ctypes.c_int)
    offs = np.ascontiguousarray(offs, np.int32)
    out = [ctypes.c_int(-1) for _ in range(4)]
    rc = L.cuvdia_plan_walk(offs.ctypes.data_as(ip), offs.size, stride, transposed, *[ctypes.byref(o) for o in out])
    return rc, tuple(o.value for o in out)


def test_window_tables_are_recognised():
    from cuv_amd import workloads as W
    # 7x7 window on a 128-wide map: 7 window rows of 7 offsets, 128 rows apart, one group; both transposes
    offs = W.window_offsets(128, 7)
    for tr in (0, 1):
        assert _walk(offs, 128 * 128, tr) == (2, (128, 7, 1, 7))
    # the same offsets in scrambled table order: the diagonals of a window row no longer sit at evenly spaced
    # table positions, which the walking kernel's addressing needs -- no window table (the products then run
    # tile by tile, as for any table)
    rng = np.random.default_rng(0)
    assert _walk(rng.permutation(offs), 128 * 128)[0] == 0
    # 5x5 window, three channel groups 64*64 rows apart; 3x3
    assert _walk(W.window_offsets(64, 5, 3), 3 * 64 * 64) == (2, (64, 5, 3, 5))
    assert _walk(W.window_offsets(192, 3), 192 * 192) == (2, (192, 3, 1, 3))
    # window tables without a walking kernel: 13x13 (the large layer), 9x9, and a 7x7 window on a map whose
    # width is no multiple of the 64-row tile
    assert _walk(W.window_offsets(256, 13, 4), 4 * 256 * 256) == (1, (256, 13, 4, 13))
    assert _walk(W.window_offsets(64, 9), 64 * 64) == (1, (64, 9, 1, 9))
    assert _walk(W.window_offsets(48, 7), 48 * 48) == (1, (48, 7, 1, 7))
    # a window that is not centred (first offset not congruent 1 mod 4 for 7 wide)
    assert _walk([dy * 128 + dx for dy in range(7) for dx in range(7)], 128 * 128)[0] == 1


def test_tables_that_are_no_window_tables():
    # a single run, runs of different lengths, a grid with a missing row, window rows at uneven distances
    assert _walk(list(range(-3, 4)), 4096)[0] == 0
    assert _walk(list(range(-3, 4)) + [100, 101], 4096)[0] == 0
    assert _walk([dy * 128 + dx for dy in (0, 1, 3) for dx in range(7)], 128 * 128)[0] == 0
    assert _walk([dy + dx for dy in (0, 128, 300) for dx in range(7)], 128 * 128)[0] == 0
    # two groups with different numbers of window rows
    assert _walk([dx for dx in range(3)] + [64 + dx for dx in range(3)] + [5000 + dx for dx in range(3)], 8192)[0] == 0
    from cuv_amd import _lib
    assert _lib.lib().cuvdia_plan_walk(None, 3, 16, 0, None, None, None, None) == _lib.EINVAL


def _walk_launch(offs, stride, h, w, batch, transposed=0):
    from cuv_amd import _lib
    offs = np.ascontiguousarray(offs, np.int32)
    ip = ctypes.POINTER(ctypes.c_int)
    return _lib.lib().cuvdia_plan_walk_launch(offs.ctypes.data_as(ip), offs.size, stride, h, w, transposed, batch)


def test_walk_launch_depends_on_the_shape_too():
    """cuvdia_plan_walk judges the table; whether a product walks also needs row counts the 64-row tiles divide,
    batch >= 24 and a launch of at least 384 workgroups."""
    from cuv_amd import _lib, workloads as W
    n = 512 * 512
    offs = W.window_offsets(512, 7)
    assert _walk(offs, n)[0] == 2
    # 512 x 512 map, batch 128: tp = 8 tiles per period, 2 column tiles -> 16 walks of 512 tiles, 32 segments each
    assert _walk_launch(offs, n, n, n, 128) == 512
    assert _walk_launch(offs, n, n, n, 128, 1) == 512
    # a narrow batch goes to the generic kernels
    assert _walk_launch(offs, n, n, n, 16) == 0
    # output rows no multiple of 64 (the table is the same, the matrix ends 40 rows early), both directions
    assert _walk(offs, n)[0] == 2
    assert _walk_launch(offs, n, n - 40, n, 128) == 0
    assert _walk_launch(offs, n, n, n - 40, 128, 1) == 0
    # ... but only the OUTPUT side needs multiples of 64; the input side multiples of 4
    assert _walk_launch(offs, n, n, n - 40, 128) > 0
    assert _walk_launch(offs, n, n, n - 42, 128) == 0
    # the headline layer's shape: 128 x 128 map, batch 128 -- too few workgroups, served tile by tile
    small = W.window_offsets(128, 7)
    assert _walk(small, 128 * 128)[0] == 2
    assert _walk_launch(small, 128 * 128, 128 * 128, 128 * 128, 128) == 0
    # no window table / no walking kernel for the window
    assert _walk_launch(list(range(-3, 4)), 4096, 4096, 4096, 128) == 0
    assert _walk_launch(W.window_offsets(256, 13, 4), 4 * 256 * 256, 4 * 256 * 256, 4 * 256 * 256, 512) == 0
    # argument errors
    assert _walk_launch(offs, n, n, n, -1) == _lib.EINVAL
    assert _walk_launch(offs, n - 8, n, n, 128) < 0          # stride shorter than the diagonals


def _window_launch(offs, stride, h, w, batch):
    from cuv_amd import _lib
    offs = np.ascontiguousarray(offs, np.int32)
    ip = ctypes.POINTER(ctypes.c_int)
    return _lib.lib().cuvdia_plan_window_launch(offs.ctypes.data_as(ip), offs.size, stride, h, w, batch)


def test_window_projection_launch_by_table_shape_and_size():
    """The projection tiled in the window's plane: tiles of 4 x 64 positions, taken from 768 (49 slots; fewer with
    two or four batch ranges per tile), 1024 (25 slots) or 1536 tiles and batch 128 (fewer slots) on; period,
    channel distances and row counts multiples of 4; chunks of 2 to 8 diagonals -- and, with a rule of their own,
    of 9 to 13."""
    from cuv_amd import _lib, workloads as W
    n = 512 * 512
    offs = W.window_offsets(512, 7)
    assert _window_launch(offs, n, n, n, 128) == 8 * 128            # 8 tile columns x 128 tile rows
    assert _window_launch(offs, n, n, n, 3) == 8 * 128              # any batch
    assert _window_launch(offs, n, n - 4, n - 8, 128) == 8 * 128    # row counts multiples of 4
    assert _window_launch(offs, n, n - 2, n, 128) == 0
    assert _window_launch(offs, n, n, n - 6, 128) == 0
    # 448-wide map: 7 x 112 = 784 tiles -- taken; 384-wide: 576 -- with two batch ranges per tile, from batch 512;
    # 256-wide: 256 -- with four, from batch 32; 192-wide: 144 -- left to the chunk-by-chunk kernel
    assert _window_launch(W.window_offsets(448, 7), 448 * 448, 448 * 448, 448 * 448, 64) == 784
    assert _window_launch(W.window_offsets(384, 7), 384 * 384, 384 * 384, 384 * 384, 64) == 0
    assert _window_launch(W.window_offsets(384, 7), 384 * 384, 384 * 384, 384 * 384, 512) == 576
    assert _window_launch(W.window_offsets(256, 7), 256 * 256, 256 * 256, 256 * 256, 32) == 256
    assert _window_launch(W.window_offsets(256, 7), 256 * 256, 256 * 256, 256 * 256, 16) == 0
    assert _window_launch(W.window_offsets(256, 5), 256 * 256, 256 * 256, 256 * 256, 1024) == 0
    assert _window_launch(W.window_offsets(192, 7), 192 * 192, 192 * 192, 192 * 192, 1024) == 0
    # 5 x 5 from 1024 tiles, 3 x 3 from 1536 and batch 128
    assert _window_launch(W.window_offsets(448, 5), 448 * 448, 448 * 448, 448 * 448, 64) == 0
    assert _window_launch(W.window_offsets(512, 5), n, n, n, 64) == 1024
    assert _window_launch(W.window_offsets(512, 3), n, n, n, 512) == 0
    assert _window_launch(W.window_offsets(640, 3), 640 * 640, 640 * 640, 640 * 640, 128) == 10 * 160
    assert _window_launch(W.window_offsets(640, 3), 640 * 640, 640 * 640, 640 * 640, 64) == 0
    # four channels of a 256-wide map: 4 tile columns x 256 tile rows x 4 groups
    offs4 = W.window_offsets(256, 7, 4)
    assert _window_launch(offs4, 4 * 256 * 256, 4 * 256 * 256, 4 * 256 * 256, 32) == 4 * 256 * 4
    # 13 window rows of 7 diagonals: two blocks of 8 window rows per tile
    tall = [dy * 512 + dx for dy in range(-6, 7) for dx in range(-3, 4)]
    assert _window_launch(tall, n, n, n, 128) == 2 * 8 * 128
    # window rows of 9 to 13 diagonals: blocks of 7 or 5 window rows (13 -> 7 + 6, 9 -> 5 + 4, 11 -> 7 + 4); on maps
    # at least 192 wide taken from 4096 workgroups, from 1024 (512 on maps at least 256 wide) when the blocks are at
    # least nine tenths full, from 1024 when window rows x channel groups are at least 22
    assert _window_launch(W.window_offsets(512, 13), n, n, n, 128) == 2 * 8 * 128
    assert _window_launch(W.window_offsets(512, 9), n, n, n, 128) == 2 * 8 * 128
    assert _window_launch(W.window_offsets(512, 11), n, n, n, 128) == 0            # 11 of 14 slots, one channel
    assert _window_launch(W.window_offsets(1024, 11), 4 * n, 4 * n, 4 * n, 32) == 2 * 16 * 256
    assert _window_launch(W.window_offsets(256, 13), 256 * 256, 256 * 256, 256 * 256, 256) == 2 * 4 * 64
    assert _window_launch(W.window_offsets(256, 9), 256 * 256, 256 * 256, 256 * 256, 256) == 2 * 4 * 64
    assert _window_launch(W.window_offsets(192, 9), 192 * 192, 192 * 192, 192 * 192, 256) == 0      # 288 workgroups
    assert _window_launch(W.window_offsets(128, 13, 4), 4 * 128 * 128, 4 * 128 * 128, 4 * 128 * 128, 256) == 0
    assert _window_launch(W.window_offsets(256, 13, 4), 4 * 256 * 256, 4 * 256 * 256, 4 * 256 * 256, 256) == 2 * 4 * 256 * 4
    assert _window_launch(W.window_offsets(256, 11, 2), 2 * 256 * 256, 2 * 256 * 256, 2 * 256 * 256, 128) == 2 * 4 * 128 * 2
    assert _window_launch(W.window_offsets(256, 15), 256 * 256, 256 * 256, 256 * 256, 64) == 0      # rows of 15
    assert _window_launch([dy * 512 + dx for dy in range(2) for dx in range(14)], n, n, n, 128) == 0   # rows of 14
    # a period that is no multiple of 4; no window table; the headline layer (64 tiles)
    assert _window_launch(W.window_offsets(510, 7), 510 * 510, 510 * 510, 510 * 510, 128) == 0
    assert _window_launch([-5, -1, 0, 1, 9], n, n, n, 128) == 0
    assert _window_launch(W.window_offsets(128, 7), 128 * 128, 128 * 128, 128 * 128, 128) == 0
    assert _lib.lib().cuvdia_plan_window_launch(None, 3, 16, 16, 16, 8) == _lib.EINVAL
