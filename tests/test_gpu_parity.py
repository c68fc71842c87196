"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle
on the same seeded inputs.

Tolerance (fp32): |gpu - oracle| <= 1e-5 * sum|terms| per element and
<= 1e-5 * max|oracle| in the max norm (see _gpu_util.assert_close_mag); the
closed-form sequence() fixtures of the reference's own tests must come out
exactly (their sums are integers below 2^24).
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def gu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import _gpu_util
    return _gpu_util


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


def _seq(rows, cols):
    return np.arange(rows * cols, dtype=np.float32).reshape(cols, rows).T.copy(order="F")


def _rand_dia(o, rng, h, w, offsets, rf=1, stride=None, pad=np.nan, lo=-1.0, hi=1.0):
    d = o.Dia(h, w, offsets, stride, rf)
    d.vals[:] = pad
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(lo, hi, int(m.sum())).astype(np.float32)
    return d


def _paths(rf):
    from cuv_amd import _lib
    return [_lib.PATH_GENERIC] if rf != 1 else [_lib.PATH_GENERIC, _lib.PATH_TILED]


# ------------------------------------------- the reference's own fixtures ---
def test_reference_spmv_fixture_exact(oracle, gu):
    # src/tests/spmv.cpp:103-143
    fx = _load("spmv_fixture.json")
    A = oracle.Dia(fx["h"], fx["w"], fx["offsets"], fx["stride"], 1)
    A.vals[:] = np.arange(A.vals.size, dtype=np.float32)
    B, C = _seq(fx["w"], fx["batch"]), _seq(fx["h"], fx["batch"])
    for path in _paths(1):
        got, ran = gu.gpu_prod(A, B, None, "n", 1.0, 0.0, path)
        assert ran == path
        assert np.array_equal(got, np.asarray(fx["AB"], np.float32))
        got, _ = gu.gpu_prod(A, C, None, "t", 1.0, 0.0, path)
        assert np.array_equal(got, np.asarray(fx["AtC"], np.float32))
        got, _ = gu.gpu_prod(A, B, C, "n", 2.0, 1.3, path)
        np.testing.assert_allclose(got, np.asarray(fx["n_alpha2_beta1p3"]), rtol=2e-6)
        got, _ = gu.gpu_prod(A, C, B, "t", 2.0, 1.3, path)
        np.testing.assert_allclose(got, np.asarray(fx["t_alpha2_beta1p3"]), rtol=2e-6)


def test_reference_dd2dia_fixture_exact(oracle, gu):
    # src/tests/densedense_to_dia.cpp:109-197 -- row_fact 4, on the device
    fx = _load("dd2dia_fixture.json")
    C = oracle.Dia(fx["h"], fx["w"], fx["offsets"], fx["stride"], fx["rf"])
    A, B = _seq(fx["h"], fx["batch"]), _seq(fx["w"], fx["batch"])
    exp = np.asarray([[np.nan if v is None else v for v in row] for row in fx["expected"]]).reshape(-1)
    valid = ~np.isnan(exp)
    got, _ = gu.gpu_dd2dia(C, A, B, 1.0, 0.0)
    assert np.array_equal(got[valid].astype(np.float64), exp[valid])
    assert np.all(got[~valid] == 0)
    assert np.array_equal(got, oracle.dd2dia_literal(C, A, B))      # dd2s_cmp_dev_host


def test_reference_dd2dia_fixture_rf1_both_paths(oracle, gu):
    fx = _load("dd2dia_fixture.json")
    C = oracle.Dia(fx["h"], fx["w"], fx["offsets"], fx["stride"], 1)
    A, B = _seq(fx["h"], fx["batch"]), _seq(fx["w"], fx["batch"])
    ref = oracle.dd2dia_literal(C, A, B)
    for path in _paths(1):
        got, ran = gu.gpu_dd2dia(C, A, B, 1.0, 0.0, path)
        assert ran == path
        assert np.array_equal(got, ref)


# ------------------------------------------------------- shapes and edges ---
SHAPES = [
    # h, w, offsets, rf, batch
    (32, 16, [-3, -2, -1, 0, 1, 2, 3], 1, 6),
    (16, 32, [0, 1, -1], 1, 70),                    # unsorted, wide, batch not a tile multiple
    (40, 40, [5, -7, 0, 39, -39], 1, 64),           # corner diagonals
    (36, 19, [-3, -2, -1, 0, 1, 2, 3], 4, 16),      # steep (generic kernels)
    (24, 12, [2, -1, 0, 4], 2, 5),
    (200, 333, list(range(-20, 21)), 1, 33),        # long run -> several chunks
    (333, 200, [-300, -64, -63, -62, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 150, 199], 1, 128),
    (1000, 1000, [0, 0, 3, 2000, -2000, 3], 1, 40), # duplicates and out-of-range offsets
    (130, 130, [1], 1, 1),
    (64, 64, [0], 1, 64),
    (700, 650, [d * 25 + e for d in range(-2, 3) for e in range(-2, 3)], 1, 96),
    # chunk pairs of the dense x dense^T projection (first shifts a multiple of 4, at most 128 here, apart)
    (512, 512, [dy * 128 + dx for dy in range(-1, 2) for dx in range(-3, 4)], 1, 40),
    (300, 300, list(range(-8, -1)) + list(range(0, 8)) + [100, 101], 1, 7),
    (260, 1000, [-200, -199, -198, -72, -71, 56, 57, 58, 59, 700], 1, 131),
    (1024, 768, [dy * 64 + dx for dy in range(-2, 3) for dx in range(0, 8)], 1, 1),
    # wide pairs (first shifts more than 128 and at most 256 apart): 256 apart on a square and on rectangular
    # matrices both ways, 192 apart, a table that mixes a narrow pair, a wide pair and a single, and one whose
    # rows end inside the last tile
    (1536, 1536, [dy * 256 + dx for dy in range(-3, 4) for dx in range(-3, 4)], 1, 72),
    (1024, 1800, [dy * 256 + dx for dy in range(-2, 3) for dx in range(-2, 3)], 1, 33),
    (1800, 1024, [dy * 256 + dx for dy in range(-2, 2) for dx in range(0, 7)], 1, 130),
    (900, 900, [dy * 192 + dx for dy in range(-2, 3) for dx in range(-3, 4)], 1, 17),
    (1111, 1300, [0, 1, 2, 64, 65, 66, 320, 321, 576, 577, 578, 1000], 1, 41),
    # pairs further apart than a band holds (the second chunk works on the rows that far above the first's):
    # window rows 512 and 1024 apart, square and rectangular both ways; a table that mixes a near pair, a far pair
    # and a single; chunks 4096 apart on a matrix with fewer rows than that; rows that end inside the last tile;
    # chunks of 3 that far apart (which stay single)
    (4096, 4096, [dy * 512 + dx for dy in range(-3, 4) for dx in range(-3, 4)], 1, 40),
    (3000, 5000, [dy * 1024 + dx for dy in range(-2, 3) for dx in range(0, 5)], 1, 33),
    (5000, 3000, [dy * 1024 + dx for dy in range(-2, 3) for dx in range(-4, 1)], 1, 64),
    (3500, 3500, [0, 1, 2, 3, 64, 65, 66, 67, 1000, 1001, 1002, 1003, 1400, 1401, 1402, 1403, 3000], 1, 72),
    (2000, 9000, [0, 1, 2, 3, 4096, 4097, 4098, 4099], 1, 17),
    (1501, 1700, [dy * 600 + dx for dy in range(-1, 2) for dx in range(0, 4)], 1, 130),
    (1500, 1700, [dy * 600 + dx for dy in range(-1, 2) for dx in range(0, 4)], 1, 130),
    (2048, 2048, [dy * 512 + dx for dy in range(-1, 2) for dx in range(-1, 2)], 1, 24),
    # window rows a multiple of the 64-row tile apart: square, rectangular both ways, a window with
    # missing rows, ragged batch
    (2048, 2048, [dy * 64 + dx for dy in range(-3, 4) for dx in range(-3, 4)], 1, 70),
    (1536, 2304, [dy * 128 + dx for dy in range(-2, 3) for dx in range(-2, 3)], 1, 130),
    (2304, 1600, [dy * 128 + dx for dy in (-3, -2, -1, 1, 2) for dx in range(-1, 2)], 1, 64),
    # window rows wider than 8: one long chunk each (13), and runs of 9 and 12 in one table
    (512, 640, [dy * 96 + dx for dy in range(-1, 2) for dx in range(-6, 7)], 1, 72),
    (768, 512, list(range(-4, 5)) + [100 + k for k in range(12)], 1, 33),
    (1280, 1280, [dy * 128 + dx for dy in range(-4, 5) for dx in range(-4, 5)], 1, 128),
    # batches wider than 4 column tiles (walked in groups of 2 column tiles): 5 tiles (groups 2, 2, 1),
    # 8 tiles with a ragged last one, 10 tiles whose last holds a single column
    (384, 384, [dy * 32 + dx for dy in range(-1, 2) for dx in range(-2, 3)], 1, 320),
    (200, 333, list(range(-20, 21)), 1, 449),
    (700, 650, [d * 25 + e for d in range(-2, 3) for e in range(-2, 3)], 1, 577),
]


@pytest.mark.parametrize("h,w,offs,rf,batch", SHAPES)
@pytest.mark.parametrize("trans", ["n", "t"])
def test_spmm_shapes(oracle, gu, h, w, offs, rf, batch, trans):
    rng = np.random.default_rng(h * 1000 + w + batch)
    A = _rand_dia(oracle, rng, h, w, offs, rf)          # NaN in every padding slot
    n_in, n_out = (h, w) if trans == "t" else (w, h)
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
    dst = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
    for path in _paths(rf):
        # beta == 0: destination starts as NaN and must come out finite
        gu.check_prod(oracle, A, B, None, trans, 1.0, 0.0, path, "beta0 path%d" % path)
        gu.check_prod(oracle, A, B, dst, trans, 0.75, -1.5, path, "scaled path%d" % path)


@pytest.mark.parametrize("h,w,offs,rf,batch", SHAPES)
def test_dd2dia_shapes(oracle, gu, h, w, offs, rf, batch):
    if h % rf:
        pytest.skip("reference loop undefined when rows are not a multiple of row_fact")
    rng = np.random.default_rng(h * 77 + w + batch)
    C = _rand_dia(oracle, rng, h, w, offs, rf, pad=np.nan)
    A = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    B = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    for path in _paths(rf):
        gu.check_dd2dia(oracle, C, A, B, 1.0 / batch, 0.9, path, "dd2dia path%d" % path)
        Cn = oracle.Dia(h, w, offs, C.stride, rf, np.full_like(C.vals, np.nan))
        gu.check_dd2dia(oracle, Cn, A, B, 1.0, 0.0, path, "dd2dia beta0 path%d" % path)


def test_leading_dimensions_and_views(oracle, gu):
    """Operands that are column slices of wider allocations (ld > rows)."""
    import torch
    from cuv_amd import dia as D, _lib
    rng = np.random.default_rng(9)
    h, w, offs, batch = 300, 260, [-5, -4, -3, 0, 1, 2, 40], 48
    A = _rand_dia(oracle, rng, h, w, offs)
    B = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    Ad = gu.make_dev_dia(A)
    ldb, ldd = w + 12, h + 20
    Bbig = torch.full((batch, ldb), float("nan"), device="cuda:0")      # the gap between columns must never be used
    Bbig[:, :w] = D.to_device_colmajor(B)
    Dbig = torch.full((batch, ldd), -7.0, device="cuda:0")
    for path in _paths(1):
        _lib.lib().cuvdia_set_path(path)
        try:
            D.prod(Dbig[:, :h], Ad, Bbig[:, :w], "n", "n", 1.0, 0.0)
        finally:
            _lib.lib().cuvdia_set_path(_lib.PATH_AUTO)
        got = D.to_host_colmajor(Dbig[:, :h])
        gu.assert_close_mag(got, oracle.prod(A, B), oracle.prod_mag(A, B), "ld view")
        assert torch.all(Dbig[:, h:] == -7.0)          # nothing past the rows was touched


@pytest.mark.parametrize("offs", [
    [dy * 128 + dx for dy in range(-1, 2) for dx in range(-3, 4)],      # chunk pairs
    list(range(-8, -1)) + list(range(0, 8)) + [100, 101],               # single chunks
    [dy * 96 + dx for dy in range(-1, 2) for dx in range(-6, 7)],       # long chunks (13)
])
def test_dd2dia_nan_in_the_gaps_around_the_operands(oracle, gu, offs):
    """The projection stages bands of B that run past a column's ends into the neighbouring column -- or, for
    the first and last batch column of the tiles at both ends of B, past the allocation.  With lda > h and
    ldb > w and NaN in every gap (and before the first, behind the last column) no stored element may see one."""
    import torch
    from cuv_amd import dia as D, _lib
    rng = np.random.default_rng(77)
    h = w = 1024                                                         # four row tiles of 256
    batch = 40
    C = _rand_dia(oracle, rng, h, w, offs)
    P = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    Q = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    ref = oracle.dd2dia(C, P, Q, 0.25, 0.9)
    mag = oracle.dd2dia_f64(oracle.Dia(h, w, offs, C.stride, 1, np.abs(np.nan_to_num(C.vals))),
                            np.abs(P), np.abs(Q), 0.25, 0.9)
    valid = oracle.valid_mask(C)

    def gapped(host, ld, lead):
        rows, cols = host.shape
        flat = torch.full((lead + cols * ld + 16,), float("nan"), device="cuda:0")
        v = flat[lead:lead + cols * ld].view(cols, ld)[:, :rows]
        v.copy_(torch.from_numpy(np.ascontiguousarray(host.T)))
        return flat, v
    for path in _paths(1):
        for lead in (0, 4, 3):                      # 16-byte aligned bases and a misaligned one
            Cd = gu.make_dev_dia(C)
            _, Pv = gapped(P, h + 8, lead)
            _, Qv = gapped(Q, w + 12, lead)
            _lib.lib().cuvdia_set_path(path)
            try:
                D.densedense_to_dia(Cd, None, Pv, Qv, 0.25, 0.9)
            finally:
                _lib.lib().cuvdia_set_path(_lib.PATH_AUTO)
            got = Cd.pull()
            assert np.isfinite(got[valid]).all(), "a NaN from a gap reached a stored element (path %d, lead %d)" % (path, lead)
            gu.assert_close_mag(got[valid], ref[valid], mag[valid], "gapped operands, path %d, lead %d" % (path, lead))
            assert np.array_equal(got[~valid].view(np.uint32), C.vals[~valid].view(np.uint32))


def test_inf_in_the_dense_operand_reaches_only_the_rows_that_use_it(oracle, gu):
    """One Inf in B: with a table whose chunks all have the table's longest length -- every 2-d window pattern --
    the tiled kernels multiply exactly the elements the matrix stores, so the Inf shows up in the result rows
    that reference its row and nowhere else, as in the generic kernels and the reference's host loop.  (Tables
    that mix chunk lengths: the next test.)"""
    from cuv_amd import _lib
    rng = np.random.default_rng(5)
    h = w = 1024
    offs = [dy * 32 + dx for dy in range(-2, 3) for dx in range(-2, 3)]
    A = _rand_dia(oracle, rng, h, w, offs)
    B = np.asfortranarray(rng.uniform(-1, 1, (w, 70)).astype(np.float32))
    B[500, 3] = np.inf
    for trans in ("n", "t"):
        ref = oracle.prod(A, B, None, trans)
        outs = {}
        for path in _paths(1):
            got, ran = gu.gpu_prod(A, B, None, trans, 1.0, 0.0, path)
            assert ran == path
            outs[path] = got
            assert np.array_equal(np.isfinite(got), np.isfinite(ref)), "path %d, %s" % (path, trans)
        fin = np.isfinite(ref)
        assert (~fin).sum() == len(offs)                 # the rows that use B[500, 3], in column 3 only
        a, b = outs[_lib.PATH_GENERIC], outs[_lib.PATH_TILED]
        np.testing.assert_allclose(a[fin], b[fin], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("offs", [list(range(-3, 4)) + [100, 101],
                                  list(range(-8, -1)) + list(range(0, 8)) + [100, 101]],
                         ids=["7+2", "7+8+2"])
@pytest.mark.parametrize("trans", ["n", "t"])
def test_non_finite_values_with_chunks_of_mixed_length(oracle, gu, offs, trans):
    """Inf and NaN in B under a table whose chunks differ in length (the kernel is built for the longest): a
    shorter chunk must run only the diagonals it has, or 0 * Inf from the dense rows next to its own would put
    NaN into result rows that do not reference them.  The masks of Inf, NaN and finite results equal the
    oracle's on every kernel family -- in the interior, in the tiles at both ends of the operand (which take
    the other body of the tiled kernel) and with beta != 0."""
    from cuv_amd import _lib
    rng = np.random.default_rng(len(offs))
    h = w = 1024
    A = _rand_dia(oracle, rng, h, w, offs)
    B = np.asfortranarray(rng.uniform(-1, 1, (w, 70)).astype(np.float32))
    dst = np.asfortranarray(rng.uniform(-1, 1, (h, 70)).astype(np.float32))
    B[600, 3] = np.inf
    B[211, 40] = np.nan
    B[2, 5] = -np.inf           # first tile
    B[1021, 6] = np.nan         # last tile
    B[130, 69] = np.inf         # the second column tile (6 valid columns)
    for alpha, beta, d in ((1.0, 0.0, None), (0.75, -1.5, dst)):
        with np.errstate(invalid="ignore"):
            ref = oracle.prod(A, B, d, trans, alpha, beta)
        assert 0 < (~np.isfinite(ref)).sum() < 5 * len(offs) + 1
        for path in _paths(1):
            got, ran = gu.gpu_prod(A, B, d, trans, alpha, beta, path)
            assert ran == path
            what = "path %d, %s, beta %g" % (path, trans, beta)
            assert np.array_equal(np.isnan(got), np.isnan(ref)), what
            assert np.array_equal(np.isposinf(got), np.isposinf(ref)), what
            assert np.array_equal(np.isneginf(got), np.isneginf(ref)), what
            fin = np.isfinite(ref)
            np.testing.assert_allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-5, err_msg=what)


@pytest.mark.parametrize("offs", [[dy * 32 + dx for dy in range(-2, 3) for dx in range(-2, 3)],
                                  list(range(-3, 4)) + [100, 101],
                                  [dy * 512 + dx for dy in range(-1, 2) for dx in range(-3, 4)]],
                         ids=["5x5 window", "7+2", "rows 512 apart"])
def test_projection_non_finite_values_reach_only_the_slots_that_use_them(oracle, gu, offs):
    """Inf and NaN in either dense operand of densedense_to_dia: a stored element (i, j) sums A[i, b] * B[j, b]
    over the batch, so a non-finite A[i0, b0] reaches the stored slots of row i0 and a non-finite B[j0, b0] those
    of column j0 -- and nothing else, although the tiled kernel also forms products for positions that hold no
    matrix element (chunk positions past a short chunk's length, band rows outside B) and drops them.  Masks of
    NaN and +-Inf over the valid slots equal the oracle's on both kernel families; padding slots keep their bits."""
    from cuv_amd import _lib
    rng = np.random.default_rng(len(offs) + 7)
    h = w = 2048
    batch = 72
    C = _rand_dia(oracle, rng, h, w, offs)
    P = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    Q = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    P[700, 5] = np.inf
    P[3, 70] = np.nan
    Q[1200, 9] = -np.inf
    Q[w - 2, 0] = np.nan
    Q[0, 33] = np.inf
    valid = oracle.valid_mask(C)
    for alpha, beta in ((1.0 / batch, 0.0), (0.5, 0.9)):
        with np.errstate(invalid="ignore"):
            ref = oracle.dd2dia(C, P, Q, alpha, beta)
        assert 0 < (~np.isfinite(ref[valid])).sum() < 6 * len(offs)
        for path in _paths(1):
            got, ran = gu.gpu_dd2dia(C, P, Q, alpha, beta, path)
            assert ran == path
            what = "path %d, beta %g" % (path, beta)
            assert np.array_equal(got[~valid].view(np.uint32), C.vals[~valid].view(np.uint32)), what
            g, r = got[valid], ref[valid]
            assert np.array_equal(np.isnan(g), np.isnan(r)), what
            assert np.array_equal(np.isposinf(g), np.isposinf(r)), what
            assert np.array_equal(np.isneginf(g), np.isneginf(r)), what
            fin = np.isfinite(r)
            np.testing.assert_allclose(g[fin], r[fin], rtol=1e-4, atol=1e-5, err_msg=what)


def test_batch_zero_and_errors(oracle, gu):
    import ctypes
    import torch
    from cuv_amd import _lib, dia as D
    L = _lib.lib()
    A = oracle.Dia(32, 16, [-1, 0, 1], 32, 1)
    Ad = gu.make_dev_dia(A)
    x = torch.zeros(4, 16, device="cuda:0")
    y = torch.zeros(4, 32, device="cuda:0")
    sp = ctypes.c_void_p(0)
    assert L.cuvdia_spmm_f32(Ad.desc, Ad.vec.data_ptr(), x.data_ptr(), 16, y.data_ptr(), 32, 0, b"n", 1.0, 0.0, sp) == 0
    assert L.cuvdia_spmm_f32(Ad.desc, Ad.vec.data_ptr(), x.data_ptr(), 16, y.data_ptr(), 32, 4, b"x", 1.0, 0.0, sp) == _lib.EINVAL
    assert L.cuvdia_spmm_f32(Ad.desc, Ad.vec.data_ptr(), x.data_ptr(), 15, y.data_ptr(), 32, 4, b"n", 1.0, 0.0, sp) == _lib.ESHAPE
    assert L.cuvdia_spmm_f32(Ad.desc, Ad.vec.data_ptr(), None, 16, y.data_ptr(), 32, 4, b"n", 1.0, 0.0, sp) == _lib.EINVAL
    assert L.cuvdia_spmm_f32(None, Ad.vec.data_ptr(), x.data_ptr(), 16, y.data_ptr(), 32, 4, b"n", 1.0, 0.0, sp) == _lib.EINVAL
    # transposed product needs B with h rows
    with pytest.raises(RuntimeError):
        D.prod(y, Ad, x, "t")
    with pytest.raises(RuntimeError):
        D.prod(y, Ad, x, "n", "t")
    d = ctypes.c_void_p()
    offs = np.array([0, 1], np.int32)
    ip = ctypes.POINTER(ctypes.c_int)
    assert L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ip), 2, 32, 16, 8, 1) == _lib.EINVAL   # stride < h and < w
    low = np.array([0, -20], np.int32)          # rows 20..31 of a stride-16 diagonal alias the next one
    assert L.cuvdia_desc_create(ctypes.byref(d), low.ctypes.data_as(ip), 2, 32, 16, 16, 1) == _lib.ESHAPE
    assert L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ip), 2, 32, 16, 16, 1) == 0
    assert L.cuvdia_desc_destroy(d) == 0
    assert L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ip), 0, 32, 16, 32, 1) == _lib.EINVAL
    assert L.cuvdia_desc_create(ctypes.byref(d), offs.ctypes.data_as(ip), 2, 32, 16, 32, 0) == _lib.EINVAL
    # a steep matrix cannot be forced onto the tiled kernels
    S = oracle.Dia(36, 19, [0, 1], 36, 4)
    Sd = gu.make_dev_dia(S)
    L.cuvdia_set_path(_lib.PATH_TILED)
    try:
        xs = torch.zeros(32, 19, device="cuda:0")
        ys = torch.zeros(32, 36, device="cuda:0")
        assert L.cuvdia_spmm_f32(Sd.desc, Sd.vec.data_ptr(), xs.data_ptr(), 19, ys.data_ptr(), 36, 32, b"n", 1.0, 0.0, sp) == _lib.EUNSUPPORTED
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)


def test_offsets_entry_points_use_the_cache(oracle, gu):
    import ctypes
    import torch
    from cuv_amd import _lib, dia as D
    L = _lib.lib()
    rng = np.random.default_rng(21)
    A = _rand_dia(oracle, rng, 128, 96, [-2, 0, 1, 30])
    B = np.asfortranarray(rng.uniform(-1, 1, (96, 32)).astype(np.float32))
    vals = torch.from_numpy(A.vals).cuda()
    Bd = D.to_device_colmajor(B)
    out = torch.full((32, 128), float("nan"), device="cuda:0")
    ip = ctypes.POINTER(ctypes.c_int)
    for _ in range(3):
        rc = L.cuvdia_spmm_offsets_f32(vals.data_ptr(), A.offsets.ctypes.data_as(ip), A.nd, A.stride, A.h, A.w, 1,
                                       Bd.data_ptr(), 96, out.data_ptr(), 128, 32, b"n", 1.0, 0.0, None)
        assert rc == 0
    torch.cuda.synchronize()
    gu.assert_close_mag(D.to_host_colmajor(out), oracle.prod(A, B), oracle.prod_mag(A, B), "offsets form")
    C = _rand_dia(oracle, rng, 128, 96, [-2, 0, 1, 30], pad=5.0)
    Ah = np.asfortranarray(rng.uniform(-1, 1, (128, 32)).astype(np.float32))
    cv = torch.from_numpy(C.vals).cuda()
    rc = L.cuvdia_dd2dia_offsets_f32(cv.data_ptr(), C.offsets.ctypes.data_as(ip), C.nd, C.stride, C.h, C.w, 1,
                                     D.to_device_colmajor(Ah).data_ptr(), 128, Bd.data_ptr(), 96, 32, 0.5, 0.25, None)
    assert rc == 0
    torch.cuda.synchronize()
    ref = oracle.dd2dia(C, Ah, B, 0.5, 0.25)
    np.testing.assert_allclose(cv.cpu().numpy(), ref, rtol=1e-5, atol=1e-6)
    assert L.cuvdia_cache_clear() == 0


# ------------------------------------------------- the measured workloads ---
def _o_dia(oracle, wl):
    p = wl.pattern
    return oracle.Dia(p.h, p.w, p.offsets, p.stride, p.rf, wl.vals)


def test_cfg0_spmv(oracle, gu):
    from cuv_amd import workloads as W
    for trans in ("n", "t"):
        wl = W.cfg0(trans)
        for path in _paths(1):
            gu.check_prod(oracle, _o_dia(oracle, wl), wl.X, None, trans, 1.0, 0.0, path, wl.name)


def test_cfg1_up_pass(oracle, gu):
    from cuv_amd import workloads as W, _lib
    wl = W.cfg1()
    _, ran = gu.check_prod(oracle, _o_dia(oracle, wl), wl.X, None, "n", 1.0, 0.0, _lib.PATH_AUTO, wl.name)
    assert ran == _lib.PATH_TILED


def test_cfg2_down_pass(oracle, gu):
    from cuv_amd import workloads as W, _lib
    wl = W.cfg2()
    _, ran = gu.check_prod(oracle, _o_dia(oracle, wl), wl.X, wl.dst, "t", 1.0, 0.5, _lib.PATH_AUTO, wl.name)
    assert ran == _lib.PATH_TILED


def test_cfg3_weight_gradient(oracle, gu):
    from cuv_amd import workloads as W, _lib
    wl = W.cfg3()
    _, ran = gu.check_dd2dia(oracle, _o_dia(oracle, wl), wl.A, wl.B, wl.alpha, wl.beta, _lib.PATH_AUTO, wl.name)
    assert ran == _lib.PATH_TILED


def test_cfg1_generic_matches_too(oracle, gu):
    from cuv_amd import workloads as W, _lib
    wl = W.cfg1()
    gu.check_prod(oracle, _o_dia(oracle, wl), wl.X[:, :16], None, "n", 1.0, 0.0, _lib.PATH_GENERIC, "cfg1 generic")
    wl3 = W.cfg3()
    gu.check_dd2dia(oracle, _o_dia(oracle, wl3), wl3.A[:, :24], wl3.B[:, :24], 1.0 / 24, 0.9, _lib.PATH_GENERIC, "cfg3 generic")


def test_cfg4_reduced_multichannel(oracle, gu):
    """The large layer's offset structure (4 channel shifts x 13x13 window) at a
    map size the oracle finishes in seconds: 64x64x4 rows, batch 72."""
    from cuv_amd import workloads as W, _lib
    for trans in ("n", "t"):
        wl = W.cfg4("spmm", trans, px=64, batch=72)
        gu.check_prod(oracle, _o_dia(oracle, wl), wl.X, None, trans, 1.0, 0.0, _lib.PATH_TILED, wl.name)
    wl = W.cfg4("dd2dia", px=64, batch=72, beta=0.9)
    gu.check_dd2dia(oracle, _o_dia(oracle, wl), wl.A, wl.B, 1.0 / 72, 0.9, _lib.PATH_TILED, wl.name)


def test_cfg4_full_size_properties(gu):
    """The large layer at its full shape (262144 rows, 4 x 13 x 13 = 676
    diagonals, batch 256; about 57 GFLOP per product), where the CPU oracle
    would take minutes.  Inputs are drawn on the device; what is checked does
    not depend on the size:
      * sampled output rows / diagonal slots against an fp64 evaluation of
        the defining sum (rows at both ends, at channel boundaries, random),
      * the generic and the tiled kernels agree on the whole result,
      * <A*X, H> == <X, A^T*H>  and  <proj(P*Q^T), W> == <W*Q, P>  in fp64,
      * padding slots (NaN) are neither read nor written.
    Tolerance: 1e-5 of the summed term magnitudes per element."""
    import torch
    from cuv_amd import dia as D, _lib, workloads as W
    L = _lib.lib()
    dev = "cuda:0"
    p = W.pattern_large(256, 4, 13)
    n, nd, batch = p.h, len(p.offsets), 256
    assert (n, nd) == (262144, 676) and p.stride == n
    g = torch.Generator(device=dev)
    g.manual_seed(0xC0FFEE + 4)
    off = torch.tensor(np.asarray(p.offsets, np.int32), device=dev)
    rows = torch.arange(n, dtype=torch.int32, device=dev)
    col = rows[None, :] + off[:, None]
    valid = (col >= 0) & (col < n)                      # (nd, n)
    del col
    assert int(valid.sum()) == 110616022

    def new_dia(fill_valid):
        m = D.dev_dia_matrix_f(n, n, nd, n, 1, device=dev)
        m.set_offsets(p.offsets)
        m.vec.copy_(torch.where(valid, fill_valid.view(nd, n), torch.full((), float("nan"), device=dev)).view(-1))
        return m

    A = new_dia(torch.randn(nd * n, generator=g, device=dev) * 0.01)
    assert A.info()["nnz"] == 110616022
    X = torch.rand(batch, n, generator=g, device=dev)
    H = torch.rand(batch, n, generator=g, device=dev)
    sample = torch.tensor(sorted(set(
        [0, 1, 5, 6, 7, 255, 256, 1541, 1542, 65535, 65536, 65537, 131071, 131072, 196608, n - 1543, n - 1542,
         n - 257, n - 7, n - 2, n - 1] + list(np.random.default_rng(4).integers(0, n, 27)))), device=dev)

    def rows_expected(M, Bm, trans):
        """fp64 value and term-magnitude sum of rows `sample` of op(M)*Bm."""
        v = torch.nan_to_num(M.vec.view(nd, n))
        if not trans:       # y[i] = sum_d v[d, i] * x[i + off_d]
            src = sample[:, None] + off[None, :]
            ok = (src >= 0) & (src < n)
            a = v[:, sample].T
        else:               # y[j] = sum_d v[d, j - off_d] * x[j - off_d]
            src = sample[:, None] - off[None, :]
            ok = (src >= 0) & (src < n)
            a = v[torch.arange(nd, device=dev)[None, :], src.clamp(0, n - 1)]
        a = (a * ok).double()
        xs = Bm[:, src.clamp(0, n - 1)].double()      # (batch, rows, nd)
        return torch.einsum("rd,crd->cr", a, xs), torch.einsum("rd,crd->cr", a.abs(), xs.abs())

    def close(got, ref, mag, what):
        assert torch.isfinite(got).all(), what
        err = (got.double() - ref).abs()
        assert bool((err <= 1e-5 * mag + 1e-30).all()), "%s: worst err/mag %.3g" % (what, float((err / (mag + 1e-30)).max()))

    def run_prod(dst, M, Bm, trans, path):
        _lib.check(L.cuvdia_set_path(path), "set_path")
        try:
            D.prod(dst, M, Bm, trans, "n", 1.0, 0.0)
            assert L.cuvdia_last_path() == path
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)

    # forward and transposed products
    Y = torch.full((batch, n), float("nan"), device=dev)
    Yt = torch.full((batch, n), float("nan"), device=dev)
    run_prod(Y, A, X, "n", _lib.PATH_TILED)
    run_prod(Yt, A, H, "t", _lib.PATH_TILED)
    for out, Bm, trans in ((Y, X, False), (Yt, H, True)):
        ref, mag = rows_expected(A, Bm, trans)
        close(out[:, sample], ref, mag, "cfg4 full %s sampled rows" % ("trans" if trans else "fwd"))
    lhs = float((Y.double() * H.double()).sum())
    rhs = float((X.double() * Yt.double()).sum())
    scale = float((Y.double().abs() * H.double()).sum())
    assert abs(lhs - rhs) <= 1e-5 * scale, ("adjoint identity", lhs, rhs, scale)
    Yg = torch.full((batch, n), float("nan"), device=dev)
    run_prod(Yg, A, X, "n", _lib.PATH_GENERIC)
    assert float((Y - Yg).abs().max()) <= 1e-5 * float(Yg.abs().max()), "tiled vs generic"
    del Yg, Yt

    # weight gradient: G = proj(X * H^T) on the pattern, beta == 0 over NaN -- through the chunk-by-chunk kernel and
    # through the kernel tiled in the window's plane, which the automatic choice takes at this size
    Y2 = torch.full((batch, n), float("nan"), device=dev)
    run_prod(Y2, A, H, "n", _lib.PATH_TILED)
    src = sample[:, None] + off[None, :]
    ok = (src >= 0) & (src < n)
    xs = X[:, sample].double()                                         # (batch, rows)
    hs = H[:, src.clamp(0, n - 1)].double()                            # (batch, rows, nd)
    ref = torch.einsum("cr,crd->dr", xs, hs) / batch
    for forced, expected in ((_lib.PATH_TILED_NOWALK, _lib.PATH_TILED), (_lib.PATH_WINDOW, _lib.PATH_WINDOW),
                             (_lib.PATH_AUTO, _lib.PATH_WINDOW)):
        G = new_dia(torch.zeros(nd * n, device=dev))
        G.vec.fill_(float("nan"))
        bd = D.dev_block_descriptor_f(G)
        _lib.check(L.cuvdia_set_path(forced), "set_path")
        try:
            D.densedense_to_dia(G, bd, X, H, 1.0 / batch, 0.0)
            assert L.cuvdia_last_path() == expected, (forced, L.cuvdia_last_kernel())
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)
        Gv = G.vec.view(nd, n)
        assert bool(torch.isnan(Gv[~valid]).all()), "padding slots were written"
        assert bool(torch.isfinite(Gv[valid]).all()), "valid slots not written"
        got = Gv[:, sample].double()
        err = (got - ref).abs()[ok.T]
        assert float(err.max()) <= 1e-5 * float(ref.abs().max()), "dd2dia sampled slots %.3g" % float(err.max())
        # <proj(X H^T)/batch, A> == <A*H', X>/batch with H' = H: sum_valid G*A == <Y2, X>/batch, Y2 = A*H
        lhs = float((torch.nan_to_num(Gv).double() * torch.nan_to_num(A.vec.view(nd, n)).double()).sum())
        rhs = float((Y2.double() * X.double()).sum()) / batch
        scale = float((Y2.double().abs() * X.double()).sum()) / batch
        assert abs(lhs - rhs) <= 1e-5 * scale, ("gradient adjoint identity", forced, lhs, rhs, scale)
        del G, Gv, bd


# ------------------------------------------------------------ avg_diagonals ---
@pytest.mark.parametrize("h,w,offs", [
    (32, 16, [-3, -2, -1, 0, 1, 2, 3]),
    (1000, 700, [0, 5, -999, 699, -400, 12]),
    (16384, 16384, [dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)]),
    (40, 40, [39, -39, 0, 100, -100]),                # single-slot and empty diagonals
])
def test_avg_diagonals(oracle, gu, h, w, offs):
    """Mean of each diagonal over its valid slots against the host loop
    (serial fp32 sum); the device sums in a different order, so the bound is
    1e-5 of the mean magnitude sum.  Padding holds NaN and must not be read."""
    import torch
    from cuv_amd import dia as D
    rng = np.random.default_rng(h + w)
    A = _rand_dia(oracle, rng, h, w, offs, 1, pad=np.nan)
    valid = oracle.valid_mask(A).reshape(len(offs), -1)
    n_valid = valid.sum(axis=1)
    ref = oracle.avg_diagonals(A)
    vals = np.nan_to_num(A.vals.reshape(len(offs), -1))
    exact = np.where(n_valid > 0, vals.astype(np.float64).sum(axis=1) / np.maximum(n_valid, 1), 0.0)
    mag = np.where(n_valid > 0, np.abs(vals).astype(np.float64).sum(axis=1) / np.maximum(n_valid, 1), 0.0)
    dev = gu.make_dev_dia(A)
    out = torch.full((len(offs),), float("nan"), dtype=torch.float32, device="cuda:0")
    D.avg_diagonals(out, dev)
    got = out.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    live = n_valid > 0
    assert np.all(np.abs(got[live] - ref[live]) <= 1e-5 * mag[live] + 1e-30)
    assert np.all(np.abs(got[live] - exact[live]) <= 1e-5 * mag[live] + 1e-30)
    assert np.all(got[~live] == 0.0)                  # the reference divides by zero there
    # sequence() data: every mean is a closed form (src/tests/dia_mat.cpp:130-140 fixture)
    S = oracle.Dia(h, w, offs, A.stride, 1)
    small = h * len(offs) < 2 ** 22
    if small:
        S.vals[:] = np.arange(S.vals.size, dtype=np.float32)
        D.avg_diagonals(out, gu.make_dev_dia(S))
        got = out.cpu().numpy()
        for d, k in enumerate(offs):
            i0, j0 = max(0, -k), max(0, k)
            n = min(h - i0, w - j0)
            if n > 0:
                assert abs(got[d] - (S.stride * d + i0 + (n - 1) / 2)) <= 1e-6 * (S.stride * d + i0 + n)


def test_avg_diagonals_errors(oracle, gu):
    import torch
    from cuv_amd import dia as D
    A = D.dev_dia_matrix_f(36, 19, 3, 36, 4)
    A.set_offsets([0, 1, -1])
    with pytest.raises(RuntimeError):
        D.avg_diagonals(torch.zeros(3, device="cuda:0"), A)
    B = D.dev_dia_matrix_f(32, 16, 3, 32, 1)
    B.set_offsets([0, 1, -1])
    with pytest.raises(RuntimeError):
        D.avg_diagonals(torch.zeros(4, device="cuda:0"), B)


# ----------------------------------------------- prod + bias + sigmoid, fused ---
@pytest.mark.parametrize("trans", ["n", "t"])
@pytest.mark.parametrize("h,w,offs,batch", [
    (32, 16, [-3, -2, -1, 0, 1, 2, 3], 6),
    (700, 650, [d * 25 + e for d in range(-2, 3) for e in range(-2, 3)], 96),
    (1024, 1024, [dy * 32 + dx for dy in range(-3, 4) for dx in range(-3, 4)], 128),
    # chunks of different lengths (the kernel variant that skips the diagonals a short chunk does not have)
    (900, 900, list(range(-8, -1)) + list(range(0, 8)) + [100, 101] + [300], 70),
    # more than 64 chunks of mixed lengths (the chunk table in four register sets)
    (1500, 1500, [o for k in range(70) for o in ((9 * k - 300,) if k % 3 else (9 * k - 300, 9 * k - 299))], 40),
])
def test_prod_bias_sigmoid(oracle, gu, h, w, offs, batch, trans):
    """dst = sigmoid(beta*dst + alpha*op(A)*B + bias) in one launch against the
    reference's three host steps (prod, matrix_plus_col, SIGM functor).
    Tolerance: the pre-activation is within 1e-5 of its term-magnitude sum, the
    logistic function has slope <= 1/4 and expf differs by a few ulp between
    the two sides: |gpu - ref| <= 0.25e-5 * mag + 4e-7."""
    import torch
    from cuv_amd import dia as D, _lib
    L = _lib.lib()
    rng = np.random.default_rng(h + 3 * w + batch)
    A = _rand_dia(oracle, rng, h, w, offs, 1)
    n_in, n_out = (h, w) if trans == "t" else (w, h)
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
    dst0 = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
    bias = rng.uniform(-2, 2, n_out).astype(np.float32)
    dev = gu.make_dev_dia(A)
    Bd = D.to_device_colmajor(B)
    bd = torch.from_numpy(bias).cuda()
    for path in (_lib.PATH_GENERIC, _lib.PATH_TILED):
        for (alpha, beta, use_bias, act) in ((1.0, 0.0, True, True), (0.5, -1.5, True, True),
                                             (1.0, 0.0, True, False), (2.0, 0.25, False, True)):
            dd = D.to_device_colmajor(dst0) if beta != 0 else torch.full((batch, n_out), float("nan"), device="cuda:0")
            _lib.check(L.cuvdia_set_path(path), "set_path")
            try:
                D.prod_bias_act(dd, dev, Bd, trans, alpha, beta, bd if use_bias else None,
                                _lib.ACT_SIGMOID if act else _lib.ACT_NONE)
                assert L.cuvdia_last_path() == path
            finally:
                L.cuvdia_set_path(_lib.PATH_AUTO)
            got = D.to_host_colmajor(dd).astype(np.float64)
            ref = oracle.prod_bias_act(A, B, dst0 if beta != 0 else None, trans, alpha, beta,
                                       bias if use_bias else None, act).astype(np.float64)
            mag = oracle.prod_mag(A, B, dst0 if beta != 0 else None, trans, alpha, beta)
            if use_bias:
                mag = mag + np.abs(bias)[:, None]
            assert np.isfinite(got).all()
            tol = (0.25e-5 * mag + 4e-7) if act else (1e-5 * mag + 1e-30)
            assert np.all(np.abs(got - ref) <= tol), (path, alpha, beta, use_bias, act,
                                                      float((np.abs(got - ref) / tol).max()))
            if act:
                assert got.min() >= 0.0 and got.max() <= 1.0


# ------------------------------------- prod + bias + sigmoid + Bernoulli sample ---
@pytest.mark.parametrize("trans", ["n", "t"])
@pytest.mark.parametrize("h,w,offs,batch", [
    (32, 16, [-3, -2, -1, 0, 1, 2, 3], 6),
    (700, 650, [d * 25 + e for d in range(-2, 3) for e in range(-2, 3)], 96),
    (1024, 1024, [dy * 32 + dx for dy in range(-3, 4) for dx in range(-3, 4)], 130),
])
def test_prod_bias_sigmoid_sample(oracle, gu, h, w, offs, batch, trans):
    """The fused layer update with sampling: dst = (p > u) with p the sigmoid of
    the biased product and u(row, col) the documented Philox4x32-10 draw.  The
    oracle applies rnd_binarize's rule (f > uniform) to its own p and the same
    u.  Both kernel families must give the oracle's bits wherever the two
    sides' p cannot straddle u (|p_ref - u| above the tolerance of the
    non-sampled test); elsewhere either value is right.  The seed must matter
    and the sample mean must follow the mean probability."""
    import torch
    from cuv_amd import dia as D, _lib
    L = _lib.lib()
    rng = np.random.default_rng(7 * h + w + batch)
    A = _rand_dia(oracle, rng, h, w, offs, 1)
    n_in, n_out = (h, w) if trans == "t" else (w, h)
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
    bias = rng.uniform(-1, 1, n_out).astype(np.float32)
    dev = gu.make_dev_dia(A)
    Bd = D.to_device_colmajor(B)
    bd = torch.from_numpy(bias).cuda()
    p_ref = oracle.prod_bias_act(A, B, None, trans, 1.0, 0.0, bias, True)
    mag = oracle.prod_mag(A, B, None, trans, 1.0, 0.0) + np.abs(bias)[:, None]
    tol = 0.25e-5 * mag + 4e-7
    results = {}
    for seed in (0, 0x9E3779B97F4A7C15):
        u = oracle.sample_uniform(n_out, batch, seed)
        ref = oracle.rnd_binarize(p_ref, u)
        decided = np.abs(p_ref.astype(np.float64) - u) > tol
        assert decided.mean() > 0.999
        for path in (_lib.PATH_GENERIC, _lib.PATH_TILED):
            dd = torch.full((batch, n_out), float("nan"), device="cuda:0")
            _lib.check(L.cuvdia_set_path(path), "set_path")
            try:
                D.prod_bias_act(dd, dev, Bd, trans, 1.0, 0.0, bd, _lib.ACT_SIGMOID_SAMPLE, seed=seed)
                assert L.cuvdia_last_path() == path
            finally:
                L.cuvdia_set_path(_lib.PATH_AUTO)
            got = D.to_host_colmajor(dd)
            assert np.all((got == 0.0) | (got == 1.0))
            assert np.array_equal(got[decided], ref[decided]), (path, seed, int((got != ref)[decided].sum()))
            results[(seed, path)] = got
        assert abs(float(ref.mean()) - float(p_ref.mean())) < 4.0 / np.sqrt(ref.size) + 1e-3
    assert not np.array_equal(results[(0, _lib.PATH_TILED)], results[(0x9E3779B97F4A7C15, _lib.PATH_TILED)])
    # the plain entry point takes no seed and refuses the sampling activation
    dd = torch.zeros((batch, n_out), device="cuda:0")
    rc = L.cuvdia_spmm_bias_act_f32(dev.desc, dev.vec.data_ptr(), Bd.data_ptr(), n_in, dd.data_ptr(), n_out, batch,
                                    trans.encode(), 1.0, 0.0, None, _lib.ACT_SIGMOID_SAMPLE, None)
    assert rc == _lib.EINVAL


# ------------------------------------------------ learn_step_weight_decay ---
@pytest.mark.parametrize("n,shift_w,shift_d", [(1, 0, 0), (7, 0, 0), (4096, 0, 0), (100003, 1, 1), (100003, 3, 2),
                                               (49 * 16384, 0, 0)])
def test_learn_step_weight_decay(oracle, n, shift_w, shift_d):
    """W = -lr*dW + (1 - lr*decay)*W (rprop.cu:341-346) against the fp32 host
    restatement; the GPU contracts alpha*dW + (beta*W) into one FMA, which
    moves a result by at most one rounding of the product: tolerance
    1e-6 * (|alpha*dW| + |beta*W|).  Aligned, equally misaligned and mutually
    misaligned arrays; elements around the arrays must stay untouched."""
    import torch
    from cuv_amd import dia as D
    rng = np.random.default_rng(n + shift_w)
    W = rng.normal(0, 0.01, n).astype(np.float32)
    dW = rng.normal(0, 1.0, n).astype(np.float32)
    lr, decay = 0.05, 0.002
    ref = oracle.learn_step_weight_decay(W, dW, lr, decay)
    bufw = torch.full((n + 16,), 123.0, device="cuda:0")
    bufd = torch.full((n + 16,), -7.0, device="cuda:0")
    wv = bufw[4 + shift_w:4 + shift_w + n]
    dv = bufd[4 + shift_d:4 + shift_d + n]
    wv.copy_(torch.from_numpy(W))
    dv.copy_(torch.from_numpy(dW))
    D.learn_step_weight_decay(wv, dv, lr, decay)
    got = wv.cpu().numpy()
    tol = 1e-6 * (np.abs(lr * dW.astype(np.float64)) + np.abs(W.astype(np.float64))) + 1e-30
    assert np.all(np.abs(got.astype(np.float64) - ref) <= tol), float((np.abs(got - ref) / tol).max())
    host = bufw.cpu().numpy()
    assert np.all(host[:4 + shift_w] == 123.0) and np.all(host[4 + shift_w + n:] == 123.0)
    assert np.array_equal(dv.cpu().numpy(), dW)


@pytest.mark.parametrize("n,shift", [(1, 0), (7, 0), (4096, 0), (100003, 1), (100003, (3, 2, 1)), (49 * 16384, 0)])
def test_learn_step_weight_decay_momentum(oracle, n, shift):
    """m = mw*m - lr*(dW + decay*W); W += m (rprop.cu:158-170) against the fp32
    host restatement.  The GPU may contract decay*W + dW and mw*m - lr*(...)
    into FMAs, each saving one rounding: tolerance 2e-6 * (|mw*m| + lr*|dW| +
    lr*decay*|W|) on m and that plus 1e-6*|W| on W.  Aligned, equally and
    mutually misaligned arrays; bytes around them stay untouched."""
    import torch
    from cuv_amd import dia as D
    sw, sm, sd = shift if isinstance(shift, tuple) else (shift, shift, shift)
    rng = np.random.default_rng(n + sw)
    W = rng.normal(0, 0.01, n).astype(np.float32)
    M = rng.normal(0, 0.01, n).astype(np.float32)
    dW = rng.normal(0, 1.0, n).astype(np.float32)
    lr, mw, decay = 0.05, 0.9, 0.002
    ref_w, ref_m = oracle.learn_step_weight_decay_momentum(W, M, dW, lr, mw, decay)
    bufs = [torch.full((n + 16,), fill, device="cuda:0") for fill in (123.0, 55.0, -7.0)]
    wv, mv, dv = (b[4 + s:4 + s + n] for b, s in zip(bufs, (sw, sm, sd)))
    for v, h in ((wv, W), (mv, M), (dv, dW)):
        v.copy_(torch.from_numpy(h))
    D.learn_step_weight_decay_momentum(wv, mv, dv, lr, mw, decay)
    W64, M64, d64 = (a.astype(np.float64) for a in (W, M, dW))
    tol_m = 2e-6 * (np.abs(mw * M64) + lr * np.abs(d64) + lr * decay * np.abs(W64)) + 1e-30
    got_m, got_w = mv.cpu().numpy(), wv.cpu().numpy()
    assert np.all(np.abs(got_m.astype(np.float64) - ref_m) <= tol_m)
    assert np.all(np.abs(got_w.astype(np.float64) - ref_w) <= tol_m + 1e-6 * np.abs(W64))
    for b, s, fill in zip(bufs, (sw, sm, sd), (123.0, 55.0, -7.0)):
        host = b.cpu().numpy()
        assert np.all(host[:4 + s] == fill) and np.all(host[4 + s + n:] == fill)
    assert np.array_equal(dv.cpu().numpy(), dW)


def test_momentum_steps_reach_the_optimum():
    """The reference's own check of this update (src/tests/optimize.cpp:89-123), on
    the device: 1000 steps on f(W) = 2 (W - optimum)^2, learnrate 0.01, momentum
    weight 1 - iter/1000, end within 0.01% of the optimum."""
    import torch
    from cuv_amd import dia as D
    g = torch.Generator(device="cpu").manual_seed(3)
    optimum = torch.rand(100, generator=g).cuda()
    W = torch.rand(100, generator=g).cuda()
    mom = torch.zeros(100, device="cuda:0")
    for it in range(1000):
        D.learn_step_weight_decay_momentum(W, mom, W - optimum, 0.01, 1.0 - it / 1000.0, 0.0, sync=False)
    torch.cuda.synchronize()
    assert not torch.isnan(W).any()
    assert torch.all(((W + 1) - (optimum + 1)).abs() <= 1e-4 * (optimum + 1))
    assert float((2 * (W - optimum) ** 2).mean()) <= 1e-4


def test_weight_update_fused_into_the_projection(oracle, gu):
    """examples/rbm/base.py:71-81: w_tmp = proj(v0*h0') ; w_tmp = -1/b*proj(v1*h1') + 1/b*w_tmp ;
    W = -lr*w_tmp + (1 - lr*cost)*W.  The same update in two projection calls
    and no w_tmp: W = (1 - lr*cost)*W + (-lr/b)*proj(v0*h0') ; W = W + (lr/b)*proj(v1*h1').
    Both sequences round differently; they must agree within 1e-5 of the
    magnitudes involved."""
    import torch
    from cuv_amd import dia as D
    rng = np.random.default_rng(99)
    h = w = 1024
    offs = [dy * 32 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    b = 64
    W0 = _rand_dia(oracle, rng, h, w, offs, 1)
    v0 = np.asfortranarray((rng.uniform(0, 1, (h, b)) < 0.5).astype(np.float32))
    h0 = np.asfortranarray(rng.uniform(0, 1, (w, b)).astype(np.float32))
    v1 = np.asfortranarray(rng.uniform(0, 1, (h, b)).astype(np.float32))
    h1 = np.asfortranarray(rng.uniform(0, 1, (w, b)).astype(np.float32))
    lr, cost = 0.1, 0.01
    v0d, h0d, v1d, h1d = (D.to_device_colmajor(x) for x in (v0, h0, v1, h1))
    # the reference's three steps, on the device
    Wa = gu.make_dev_dia(W0)
    tmp = gu.make_dev_dia(W0)
    bd = D.dev_block_descriptor_f(tmp)
    D.densedense_to_dia(tmp, bd, v0d, h0d, 1.0, 0.0)
    D.densedense_to_dia(tmp, bd, v1d, h1d, -1.0 / b, 1.0 / b)
    D.learn_step_weight_decay(Wa, tmp, lr, cost)
    # fused
    Wb = gu.make_dev_dia(W0)
    bdb = D.dev_block_descriptor_f(Wb)
    D.densedense_to_dia(Wb, bdb, v0d, h0d, -lr / b, 1.0 - lr * cost)
    D.densedense_to_dia(Wb, bdb, v1d, h1d, lr / b, 1.0)
    a = Wa.vec.cpu().numpy().astype(np.float64)
    c = Wb.vec.cpu().numpy().astype(np.float64)
    mask = oracle.valid_mask(W0).reshape(-1)
    g0 = np.abs(oracle.dd2dia_f64(W0, v0, h0, 1.0, 0.0)).reshape(-1)
    g1 = np.abs(oracle.dd2dia_f64(W0, v1, h1, 1.0, 0.0)).reshape(-1)
    mag = np.abs(W0.vals.astype(np.float64)) + lr / b * (g0 + g1)
    assert np.all(np.abs(a - c)[mask] <= 1e-5 * mag[mask] + 1e-30), float((np.abs(a - c)[mask] / (1e-5 * mag[mask] + 1e-30)).max())
    # and against the oracle's three host steps
    t = oracle.dd2dia(W0, v0, h0, 1.0, 0.0)
    T = oracle.Dia(h, w, offs, vals=t)
    t = oracle.dd2dia(T, v1, h1, -1.0 / b, 1.0 / b)
    ref = oracle.learn_step_weight_decay(W0.vals, t.reshape(-1), lr, cost).astype(np.float64)
    assert np.all(np.abs(a - ref)[mask] <= 1e-5 * mag[mask] + 1e-30)


def test_dia_file_round_trip_device(oracle, gu, tmp_path):
    """save_dia / load_dia: a device matrix written and read back gives the
    same product bit for bit."""
    import torch
    from cuv_amd import dia as D, io
    rng = np.random.default_rng(11)
    A = _rand_dia(oracle, rng, 300, 280, [-7, -1, 0, 1, 2, 40], 1)
    dev = gu.make_dev_dia(A)
    path = str(tmp_path / "a.npz")
    io.save_dia(path, dev)
    back = io.load_dia(path)
    assert (back.h, back.w, back.num_dia, back.stride, back.row_fact) == (dev.h, dev.w, dev.num_dia, dev.stride, dev.row_fact)
    assert np.array_equal(back.get_offsets(), dev.get_offsets())
    assert torch.equal(back.vec.view(torch.int32), dev.vec.view(torch.int32))     # padding holds NaN: compare bits
    B = D.to_device_colmajor(np.asfortranarray(rng.uniform(-1, 1, (280, 40)).astype(np.float32)))
    y0 = torch.zeros((40, 300), device="cuda:0")
    y1 = torch.zeros((40, 300), device="cuda:0")
    D.prod(y0, dev, B)
    D.prod(y1, back, B)
    assert torch.equal(y0, y1)


# --------------------------------------------------- streams and HIP graphs ---
def _layer_state(oracle, rng, n=2048, batch=96):
    import torch
    from cuv_amd import dia as D
    offs = [dy * 64 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    host = _rand_dia(oracle, rng, n, n, offs, pad=0.0, lo=-0.05, hi=0.05)

    def dev():
        m = D.dev_dia_matrix_f(n, n, len(offs), host.stride)
        m.set_offsets(host.offsets)
        return m

    W, G, M = dev().push(host.vals), dev(), dev()
    for m in (W, G, M):
        m.desc                                             # descriptors are built outside any capture
    v0 = torch.from_numpy((rng.random((batch, n)) < 0.3).astype(np.float32)).cuda()
    return dict(W=W, G=G, M=M, v0=v0, h0=torch.empty(batch, n, device="cuda:0"),
                v1=torch.empty(batch, n, device="cuda:0"), bias=torch.zeros(n, device="cuda:0"))


def _cd_step(s, seed):
    """One contrastive-divergence-shaped pass over a DIA layer: sampled up-pass,
    down-pass, gradient, momentum step; every call on the current stream."""
    from cuv_amd import _lib, dia as D
    D.prod_bias_act(s["h0"], s["W"], s["v0"], "n", 1.0, 0.0, s["bias"], _lib.ACT_SIGMOID_SAMPLE, seed, sync=False)
    D.prod_bias_act(s["v1"], s["W"], s["h0"], "t", 1.0, 0.0, s["bias"], _lib.ACT_SIGMOID, sync=False)
    D.densedense_to_dia(s["G"], None, s["h0"], s["v0"], -1.0 / s["v0"].shape[0], 0.0, sync=False)
    D.densedense_to_dia(s["G"], None, s["h0"], s["v1"], 1.0 / s["v0"].shape[0], 1.0, sync=False)
    D.learn_step_weight_decay_momentum(s["W"], s["M"], s["G"], 0.1, 0.5, 0.001, sync=False)


def test_graph_replays_match_eager_calls(oracle):
    """The entry points only launch kernels on the caller's stream, so a
    training pass can be captured into a HIP graph.  Three replays, with eager
    work and synchronisations of the program between them, must each leave
    exactly the state the same calls made eagerly leave."""
    import torch
    eager = _layer_state(oracle, np.random.default_rng(77))
    graph = _layer_state(oracle, np.random.default_rng(77))
    assert torch.equal(eager["W"].vec, graph["W"].vec) and torch.equal(eager["v0"], graph["v0"])
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _cd_step(graph, 5)                                 # warm-up on the capture stream, outside the graph
    side.synchronize()
    _cd_step(eager, 5)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        _cd_step(graph, 5)
    for replay in range(3):
        g.replay()
        _cd_step(eager, 5)
        torch.cuda.synchronize()
        filler = torch.rand(1 << 20, device="cuda:0").sum().item()      # unrelated eager work between replays
        assert filler > 0
        for k in ("h0", "v1"):
            assert torch.equal(eager[k], graph[k]), (replay, k)
        for k in ("W", "G", "M"):
            assert torch.equal(eager[k].vec, graph[k].vec), (replay, k)
    assert float(graph["M"].vec.abs().max()) > 0


def test_calls_run_on_the_callers_stream(oracle):
    """Work is ordered with the stream handed in, not with the null stream: a
    product issued on a side stream right behind a long-running fill of its
    operand on that stream sees the filled operand."""
    import torch
    from cuv_amd import dia as D
    rng = np.random.default_rng(9)
    A = _rand_dia(oracle, rng, 4096, 4096, list(range(-3, 4)), pad=0.0)
    dA = D.dev_dia_matrix_f(4096, 4096, 7, A.stride)
    dA.set_offsets(A.offsets)
    dA.push(A.vals)
    dA.desc
    side = torch.cuda.Stream()
    B = torch.zeros(64, 4096, device="cuda:0")
    dst = torch.full((64, 4096), float("nan"), device="cuda:0")
    big = torch.empty(1 << 28, device="cuda:0")
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(4):
            big.fill_(1.0)                                 # keeps the side stream busy for a while
        B.fill_(1.0)
        D.prod(dst, dA, B, "n", "n", 1.0, 0.0, sync=False)
    side.synchronize()
    ref = oracle.prod(A, np.ones((4096, 64), np.float32, order="F"), None, "n", 1.0, 0.0)
    got = D.to_host_colmajor(dst)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-6)
