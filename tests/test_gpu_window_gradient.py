"""The window-table projection kernel against the CPU oracle.

Window tables (k window rows of up to 8 consecutive diagonals, `period` rows apart) whose tiles fill the chip
are served by workgroups that own a tile of 4 x 64 positions of the window's plane.  The tests force that
kernel (CUVDIA_PATH_WINDOW) on sizes the oracle finishes in seconds, with NaN in every
padding slot of the destination, and check what the automatic choice does on both sides of its size rule and
that tables the kernel does not serve are refused when it is forced.  Tolerance: the fp32 bar of
_gpu_util.assert_close_mag (1e-5 of the sum of |terms| per element).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import _gpu_util
    return _gpu_util


def _dia(o, rng, h, w, offsets, stride=None):
    d = o.Dia(h, w, np.asarray(offsets, np.int32), stride, 1)
    d.vals[:] = np.nan
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    return d


def _operands(rng, C, batch):
    A = np.asfortranarray(rng.uniform(-1, 1, (C.h, batch)).astype(np.float32))
    B = np.asfortranarray(rng.uniform(-1, 1, (C.w, batch)).astype(np.float32))
    return A, B


def _last_kernel():
    from cuv_amd import _lib
    return _lib.lib().cuvdia_last_kernel().decode()


def _window(px, rows, cols, first_dy, first_dx, channels=1, map_elems=None):
    map_elems = px * px if map_elems is None else map_elems
    return [c * map_elems + (first_dy + dy) * px + first_dx + dx
            for c in range(channels) for dy in range(rows) for dx in range(cols)]


# px (period), rows of A, rows of B, window rows x columns, first dy, first dx, channels, batch
CASES = [
    (64, 64 * 12, 64 * 12, 7, 7, -3, -3, 1, 8),        # the centred 7 x 7, one tile column
    (128, 128 * 9, 128 * 9, 7, 7, -3, -3, 1, 13),      # two tile columns, a last tile row of one map row, a ragged batch
    (72, 72 * 10, 72 * 10, 5, 5, -2, -2, 1, 22),       # a narrower last tile column
    (64, 64 * 8, 64 * 8, 3, 3, -1, -1, 1, 3),          # less than one group of columns
    (64, 64 * 8, 64 * 11, 4, 8, 0, 0, 1, 16),          # chunks of 8, window rows all below, a wider B
    (64, 64 * 11, 64 * 8, 2, 6, -1, -5, 1, 16),        # a taller A, alignment shift 3
    (96, 96 * 8, 96 * 8, 11, 3, -5, -1, 1, 8),         # 11 window rows: two blocks of window rows
    (64, 64 * 16, 64 * 16, 7, 7, -3, -3, 2, 8),        # two groups (channels)
    (64, 64 * 12 - 4, 64 * 12 - 8, 5, 7, -2, -3, 1, 8),    # row counts that end inside a map row
    (64, 64 * 1600, 64 * 1600, 7, 7, -3, -3, 1, 9),    # 400 tiles: two batch ranges per workgroup (the cases above: four)
    (64, 64 * 3200, 64 * 3200, 7, 7, -3, -3, 1, 5),    # 800 tiles: one
    # window rows of 9 to 13 diagonals: a wave per window row, blocks of 7 window rows
    (64, 64 * 14, 64 * 14, 13, 13, -6, -6, 1, 9),      # the centred 13 x 13: two blocks (7 + 6 rows), a ragged batch
    (96, 96 * 24, 96 * 24, 9, 11, -4, -5, 2, 20),      # two groups, a narrower last tile column
    (128, 128 * 10, 128 * 12, 8, 10, -3, -2, 1, 5),    # 7 + 1 window rows, a wider B, less than one group of columns
    (64, 64 * 20 - 4, 64 * 20 - 8, 15, 12, -7, -6, 1, 17),     # three blocks, row counts that end inside a map row
    (72, 72 * 9, 72 * 9, 3, 9, -1, -8, 1, 8),          # fewer window rows than waves, all shifts but one to the left
]


@pytest.mark.parametrize("px,h,w,rows,cols,dy0,dx0,channels,batch", CASES)
def test_window_projection_matches_the_oracle(oracle, gu, px, h, w, rows, cols, dy0, dx0, channels, batch):
    from cuv_amd import _lib
    rng = np.random.default_rng(px + h + w + rows * 7 + cols + batch)
    offsets = _window(px, rows, cols, dy0, dx0, channels, map_elems=(h // channels) // 4 * 4)
    C = _dia(oracle, rng, h, w, offsets)
    A, B = _operands(rng, C, batch)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0, 0.0, _lib.PATH_WINDOW, "window beta0")
    name = "dd2dia_window_kernel<%d," if cols <= 8 else "dd2dia_window_long_kernel<%d,"
    assert ran == _lib.PATH_WINDOW and _last_kernel().startswith(name % cols)
    tiles = -(-px // 64) * -(-(-(-h // px)) // 4) * -(-rows // 8) * channels
    assert _last_kernel().endswith(", %d>" % (1 if tiles >= 768 else 2 if tiles >= 384 else 4)) or cols != 7 or rows != 7
    C.vals[oracle.valid_mask(C)] = rng.uniform(-1, 1, int(oracle.valid_mask(C).sum())).astype(np.float32)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0 / batch, 0.9, _lib.PATH_WINDOW, "window scaled")
    assert ran == _lib.PATH_WINDOW


@pytest.mark.parametrize("fs", [7, 13])
def test_window_projection_with_padded_operands_and_a_table_in_descending_order(oracle, gu, fs):
    """Leading dimensions larger than the row counts (rows of the next column follow a column's last row at a
    distance), and the offsets listed from the last to the first."""
    import torch
    from cuv_amd import _lib, dia as D
    rng = np.random.default_rng(11)
    px, n, batch = 64, 64 * (fs + 3), 12
    offsets = _window(px, fs, fs, -(fs // 2), -(fs // 2))[::-1]
    C = _dia(oracle, rng, n, n, offsets)
    A, B = _operands(rng, C, batch)
    ref = oracle.dd2dia(C, A, B, 0.5, 0.0)
    L = _lib.lib()
    Cd = gu.make_dev_dia(C)
    lda, ldb = n + 12, n + 20
    Ad = torch.full((batch + 2, lda), float("nan"), dtype=torch.float32, device="cuda:0")
    Bd = torch.full((batch + 2, ldb), float("nan"), dtype=torch.float32, device="cuda:0")
    Ad[1:batch + 1, :n] = D.to_device_colmajor(A)
    Bd[1:batch + 1, :n] = D.to_device_colmajor(B)
    L.cuvdia_set_path(_lib.PATH_WINDOW)
    try:
        D.densedense_to_dia(Cd, D.dev_block_descriptor_f(Cd), Ad[1:batch + 1, :n], Bd[1:batch + 1, :n], 0.5, 0.0)
        assert L.cuvdia_last_path() == _lib.PATH_WINDOW
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    got = Cd.pull()
    valid = oracle.valid_mask(C)
    mag = oracle.dd2dia_f64(type(C)(C.h, C.w, C.offsets, C.stride, C.rf, np.abs(C.vals)), np.abs(A), np.abs(B), 0.5, 0.0)
    gu.assert_close_mag(got[valid], ref[valid], mag[valid], "padded operands")
    assert np.isnan(got[~valid]).all()


@pytest.mark.parametrize("fs", [7, 11])
def test_non_finite_values_stay_in_the_slots_that_use_them(oracle, gu, fs):
    """An infinity in A and a NaN in B reach exactly the slots whose sums contain them."""
    from cuv_amd import _lib
    rng = np.random.default_rng(3)
    px, n, batch = 64, 64 * (fs + 2), 8
    C = _dia(oracle, rng, n, n, _window(px, fs, fs, -(fs // 2), -(fs // 2)))
    A, B = _operands(rng, C, batch)
    A[5 * px + 17, 3] = np.inf
    B[2 * px + 40, 6] = np.nan
    B[0, 0] = np.inf
    A[n - 1, batch - 1] = -np.inf
    got, ran = gu.gpu_dd2dia(C, A, B, 1.0, 0.0, _lib.PATH_WINDOW)
    assert ran == _lib.PATH_WINDOW
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.dd2dia(C, A, B, 1.0, 0.0)
    valid = oracle.valid_mask(C)
    fin = np.isfinite(ref) & valid
    assert np.array_equal(np.isnan(got[valid]), np.isnan(ref[valid]))
    assert np.array_equal(np.isposinf(got[valid]), np.isposinf(ref[valid]))
    assert np.array_equal(np.isneginf(got[valid]), np.isneginf(ref[valid]))
    assert (~np.isfinite(ref[valid])).sum() > 0
    np.testing.assert_allclose(got[fin], ref[fin], rtol=0, atol=1e-4)


def test_the_choice_by_size_and_the_refusals(oracle, gu):
    from cuv_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(21)
    # 1024 tiles of a 5 x 5 window: taken by size
    px, n, batch = 256, 256 * 1024, 4
    C = _dia(oracle, rng, n, n, _window(px, 5, 5, -2, -2))
    A, B = _operands(rng, C, batch)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0, 0.0, _lib.PATH_AUTO, "taken by size")
    assert ran == _lib.PATH_WINDOW and _last_kernel().startswith("dd2dia_window_kernel<5,")
    # as many tiles of a 3 x 3 window at a small batch: not taken
    C = _dia(oracle, rng, n, n, _window(px, 3, 3, -1, -1))
    A, B = _operands(rng, C, batch)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0, 0.0, _lib.PATH_AUTO, "small window, small batch")
    assert ran == _lib.PATH_TILED
    # the same table on fewer rows: left to the chunk-by-chunk kernel, which agrees
    n = 256 * 64
    C = _dia(oracle, rng, n, n, _window(px, 3, 3, -1, -1))
    A, B = _operands(rng, C, batch)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0, 0.0, _lib.PATH_AUTO, "left alone")
    assert ran == _lib.PATH_TILED and _last_kernel().startswith("dd2dia_tiled_kernel")
    # 256 tiles of a 7 x 7 window at batch 32: taken with four batch ranges per workgroup
    n = 64 * 1024
    C = _dia(oracle, rng, n, n, _window(64, 7, 7, -3, -3))
    A, B = _operands(rng, C, 32)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 1.0 / 32, 0.9, _lib.PATH_AUTO, "four ranges")
    assert ran == _lib.PATH_WINDOW and _last_kernel() == "dd2dia_window_kernel<7, 1, 4>"
    n = 256 * 64
    # window rows of 9 to 13 diagonals: 512 workgroups of a 13 x 13 or a 9 x 9 window on a 256-wide map are taken
    # (blocks of 7 and of 5 window rows), of an 11 x 11 (11 of 14 wave slots) not
    n = 256 * 256
    C = _dia(oracle, rng, n, n, _window(256, 13, 13, -6, -6))
    A, B = _operands(rng, C, 4)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 0.25, 0.9, _lib.PATH_AUTO, "long rows taken by size")
    assert ran == _lib.PATH_WINDOW and _last_kernel() == "dd2dia_window_long_kernel<13, 2, 7>"
    C = _dia(oracle, rng, n, n, _window(256, 9, 9, -4, -4))
    A, B = _operands(rng, C, 4)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 0.25, 0.9, _lib.PATH_AUTO, "9 rows: blocks of 5")
    assert ran == _lib.PATH_WINDOW and _last_kernel() == "dd2dia_window_long_kernel<9, 0, 5>"
    C = _dia(oracle, rng, n, n, _window(256, 11, 11, -5, -5))
    A, B = _operands(rng, C, 4)
    _, ran = gu.check_dd2dia(oracle, C, A, B, 0.25, 0.9, _lib.PATH_AUTO, "long rows left alone")
    assert ran == _lib.PATH_TILED and _last_kernel().startswith("dd2dia_tiled_kernel<11,")
    n = 256 * 64
    # forced on what it does not serve: window rows of 14 diagonals, a period that is no multiple of 4, no window table
    for offsets, b in ((_window(256, 2, 14, -1, -7), 8), (_window(254, 3, 3, -1, -1), 8), ([-5, -1, 0, 1, 9], 8)):
        C = _dia(oracle, rng, n, n, offsets)
        A, B = _operands(rng, C, b)
        Cd = gu.make_dev_dia(C)
        from cuv_amd import dia as D
        Ad, Bd = D.to_device_colmajor(A), D.to_device_colmajor(B)
        L.cuvdia_set_path(_lib.PATH_WINDOW)
        try:
            with pytest.raises(_lib.CuvDiaError) as err:
                D.densedense_to_dia(Cd, D.dev_block_descriptor_f(Cd), Ad, Bd, 1.0, 0.0)
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)
        assert err.value.code == _lib.EUNSUPPORTED


@pytest.mark.parametrize("seed", range(16))
def test_random_window_shapes(oracle, gu, seed):
    """Seeded window tables nobody picked by hand: period, window, first shift, channel groups, row counts and batch
    drawn at random within what the kernel serves."""
    from cuv_amd import _lib
    rng = np.random.default_rng(1000 + seed)
    px = 4 * int(rng.integers(16, 50)) if seed % 4 else 4 * int(rng.integers(5, 16))     # (some maps narrower than a tile)
    rows, cols = int(rng.integers(2, 12)), int(rng.integers(2, 9))
    dy0, dx0 = -int(rng.integers(0, rows)), -int(rng.integers(0, cols))
    channels = int(rng.choice([1, 1, 2, 3]))
    map_rows = rows + int(rng.integers(4, 12))
    map_elems = px * map_rows
    h = channels * map_elems - 4 * int(rng.integers(0, 3))
    w = channels * map_elems - 4 * int(rng.integers(0, 3))
    batch = int(rng.choice([1, 3, 4, 7, 8, 17, 32]))
    offsets = _window(px, rows, cols, dy0, dx0, channels, map_elems)
    if seed % 3 == 0:
        offsets = offsets[::-1]                                        # listed from the last to the first
    stride = max(h, w) + int(rng.choice([0, 0, 1, 3, 4, 13]))         # (a stride that is no multiple of 4: the 16-byte
    C = _dia(oracle, rng, h, w, offsets, stride)                       # stores then start at any 4-byte boundary)
    A, B = _operands(rng, C, batch)
    alpha, beta = float(rng.choice([1.0, -0.5, 1.0 / batch])), float(rng.choice([0.0, 0.9, -1.5]))
    _, ran = gu.check_dd2dia(oracle, C, A, B, alpha, beta, _lib.PATH_WINDOW, "random window %d" % seed)
    assert ran == _lib.PATH_WINDOW


@pytest.mark.parametrize("seed", range(12))
def test_random_window_shapes_with_rows_of_9_to_13_diagonals(oracle, gu, seed):
    """The same draw for the kernel that serves rows of 9 to 13 diagonals (a wave per window row)."""
    from cuv_amd import _lib
    rng = np.random.default_rng(2000 + seed)
    px = 4 * int(rng.integers(16, 60)) if seed % 4 else 4 * int(rng.integers(5, 16))
    rows, cols = int(rng.integers(1, 16)), int(rng.integers(9, 14))
    dy0, dx0 = -int(rng.integers(0, rows)), -int(rng.integers(0, cols))
    channels = int(rng.choice([1, 1, 2, 3]))
    map_elems = px * (rows + int(rng.integers(4, 12)))
    h = channels * map_elems - 4 * int(rng.integers(0, 3))
    w = channels * map_elems - 4 * int(rng.integers(0, 3))
    batch = int(rng.choice([1, 3, 7, 8, 9, 17, 32, 50]))
    offsets = _window(px, rows, cols, dy0, dx0, channels, map_elems)
    if seed % 3 == 0:
        offsets = offsets[::-1]
    stride = max(h, w) + int(rng.choice([0, 0, 1, 3, 4, 13]))
    C = _dia(oracle, rng, h, w, offsets, stride)
    A, B = _operands(rng, C, batch)
    alpha, beta = float(rng.choice([1.0, -0.5, 1.0 / batch])), float(rng.choice([0.0, 0.9, -1.5]))
    _, ran = gu.check_dd2dia(oracle, C, A, B, alpha, beta, _lib.PATH_WINDOW, "random long rows %d" % seed)
    assert ran == _lib.PATH_WINDOW and _last_kernel().startswith("dd2dia_window_long_kernel<%d," % cols)


def test_a_sweep_size_against_sampled_exact_sums_and_the_chunk_kernel(gu):
    """512 x 512 map, 7 x 7 window, batch 32 -- a size the automatic choice gives to this kernel and the oracle
    would take minutes for: 4000 stored slots drawn at random are compared with their sums in fp64, the padding
    slots must keep their NaN, and the whole result must lie within rounding of the chunk-by-chunk kernel's."""
    import torch
    from cuv_amd import _lib, dia as D, workloads as W
    rng = np.random.default_rng(7)
    px, batch = 512, 32
    n = px * px
    offs = W.window_offsets(px, 7)
    A = np.asfortranarray(rng.uniform(-1, 1, (n, batch)).astype(np.float32))
    B = np.asfortranarray(rng.uniform(-1, 1, (n, batch)).astype(np.float32))
    Ad, Bd = D.to_device_colmajor(A), D.to_device_colmajor(B)
    L = _lib.lib()
    results = {}
    for path in (_lib.PATH_AUTO, _lib.PATH_TILED_NOWALK):
        C = D.dev_dia_matrix_f(n, n, len(offs), n, 1, device="cuda:0")
        C.set_offsets(offs)
        C.vec.fill_(float("nan"))
        L.cuvdia_set_path(path)
        try:
            D.densedense_to_dia(C, D.dev_block_descriptor_f(C), Ad, Bd, 0.5, 0.0)
            ran = L.cuvdia_last_path()
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)
        results[path] = (C.pull().reshape(len(offs), n), ran)
    got, ran = results[_lib.PATH_AUTO]
    assert ran == _lib.PATH_WINDOW
    other, ran = results[_lib.PATH_TILED_NOWALK]
    assert ran == _lib.PATH_TILED
    i = np.arange(n)
    valid = np.stack([(i + k >= 0) & (i + k < n) for k in offs])
    assert np.isnan(got[~valid]).all() and np.isfinite(got[valid]).all()
    # every term is below 1 in magnitude: 1e-5 of the batch bounds 1e-5 of the sum of |terms|
    assert np.abs(got[valid] - other[valid]).max() <= 1e-5 * 0.5 * batch
    d = rng.integers(0, len(offs), 4000)
    r = rng.integers(0, n, 4000)
    keep = valid[d, r]
    d, r = d[keep], r[keep]
    exact = 0.5 * np.einsum("ij,ij->i", A[r].astype(np.float64), B[r + offs[d]].astype(np.float64))
    mag = 0.5 * np.einsum("ij,ij->i", np.abs(A[r]).astype(np.float64), np.abs(B[r + offs[d]]).astype(np.float64))
    assert (np.abs(got[d, r] - exact) <= 1e-5 * mag + 1e-30).all()


def test_window_projection_under_graph_capture_and_replay(oracle, gu):
    """The kernel recorded into a HIP graph and replayed with the program's own eager work between the replays:
    every replay equals the eager result (beta != 0: the destination is restored before each replay)."""
    import torch
    from cuv_amd import dia as D, _lib
    rng = np.random.default_rng(12)
    px, n, batch = 64, 64 * 12, 20
    C = _dia(oracle, rng, n, n, _window(px, 5, 5, -2, -2))
    A, B = _operands(rng, C, batch)
    Ad, Bd = D.to_device_colmajor(A), D.to_device_colmajor(B)
    L = _lib.lib()
    L.cuvdia_set_path(_lib.PATH_WINDOW)
    try:
        Ce = gu.make_dev_dia(C)
        start = Ce.vec.clone()
        D.densedense_to_dia(Ce, D.dev_block_descriptor_f(Ce), Ad, Bd, 0.25, 0.9)
        assert L.cuvdia_last_path() == _lib.PATH_WINDOW
        eager = Ce.vec.clone()
        Cg = gu.make_dev_dia(C)
        bd = D.dev_block_descriptor_f(Cg)
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            D.densedense_to_dia(Cg, bd, Ad, Bd, 0.25, 0.9, sync=False)      # warm-up on a side stream
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            D.densedense_to_dia(Cg, bd, Ad, Bd, 0.25, 0.9, sync=False)
        for rep in range(3):
            Cg.vec.copy_(start)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(Cg.vec.view(torch.int32), eager.view(torch.int32)), "replay %d differs from the eager call" % rep
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    ref = oracle.dd2dia(C, A, B, 0.25, 0.9)
    valid = oracle.valid_mask(C)
    mag = oracle.dd2dia_f64(type(C)(C.h, C.w, C.offsets, C.stride, C.rf, np.abs(C.vals)), np.abs(A), np.abs(B), 0.25, 0.9)
    gu.assert_close_mag(eager.cpu().numpy()[valid], ref[valid], mag[valid], "eager")
