"""The walking SpMM kernel against the CPU oracle.

Window tables (k window rows of k consecutive diagonals, `period` rows apart,
period a multiple of the 64-row tile) on products of many tiles are served by
workgroups that walk down the rows and keep k tiles alive.  The tests force
that kernel on sizes the oracle finishes in seconds, with NaN in every padding
slot of the matrix and in the destination when beta == 0, and check that the
automatic choice takes it on a product that is large enough and leaves it
alone where its shape conditions do not hold.  Tolerance: the fp32 bar of
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


def _window_dia(o, rng, h, w, px, fs, channels=1):
    from cuv_amd import workloads as W
    d = o.Dia(h, w, W.window_offsets(px, fs, channels), None, 1)
    d.vals[:] = np.nan
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    return d


def _operands(rng, A, batch, trans):
    n_in, n_out = (A.h, A.w) if trans == "t" else (A.w, A.h)
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
    dst = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
    return B, dst


# px, window, channels, batch: one and several segments per walk, a ragged last column tile, two residues
# per period (px 128), several groups (channels)
WALK_CASES = [
    (64, 7, 1, 64),
    (64, 7, 1, 70),
    (128, 7, 1, 33),
    (64, 5, 1, 130),
    (64, 3, 1, 64),
    (64, 7, 2, 64),
    (64, 5, 3, 17),
]


@pytest.mark.parametrize("px,fs,channels,batch", WALK_CASES)
@pytest.mark.parametrize("trans", ["n", "t"])
def test_walk_matches_the_oracle(oracle, gu, px, fs, channels, batch, trans):
    from cuv_amd import _lib
    rng = np.random.default_rng(px * 100 + fs * 10 + channels + batch)
    n = px * px * channels
    A = _window_dia(oracle, rng, n, n, px, fs, channels)
    B, dst = _operands(rng, A, batch, trans)
    _, ran = gu.check_prod(oracle, A, B, None, trans, 1.0, 0.0, _lib.PATH_WALK, "walk beta0")
    assert ran == _lib.PATH_WALK
    _, ran = gu.check_prod(oracle, A, B, dst, trans, 0.75, -1.5, _lib.PATH_WALK, "walk scaled")
    assert ran == _lib.PATH_WALK


@pytest.mark.parametrize("px,fs,channels,batch", [(64, 7, 1, 70), (128, 5, 1, 33), (64, 3, 2, 64)])
@pytest.mark.parametrize("trans", ["n", "t"])
def test_walk_with_bias_and_sigmoid_at_the_tiles_exit(oracle, gu, px, fs, channels, batch, trans):
    """dst = sigmoid(beta*dst + alpha*op(A)*B + bias) through the walking kernel against the reference's three host
    steps, and the sampled form against the oracle's draw.  Tolerances as for the tile-by-tile kernel: 0.25e-5 *
    magnitude + 4e-7 behind the sigmoid, 1e-5 * magnitude without."""
    import torch
    from cuv_amd import dia as D, _lib
    L = _lib.lib()
    rng = np.random.default_rng(px + fs + channels + batch)
    n = px * px * channels
    A = _window_dia(oracle, rng, n, n, px, fs, channels)
    B, dst0 = _operands(rng, A, batch, trans)
    bias = rng.uniform(-2, 2, n).astype(np.float32)
    dev = gu.make_dev_dia(A)
    Bd = D.to_device_colmajor(B)
    bd = torch.from_numpy(bias).cuda()
    for (alpha, beta, use_bias, act) in ((1.0, 0.0, True, True), (0.5, -1.5, True, True), (1.0, 0.0, True, False),
                                         (2.0, 0.25, False, True)):
        dd = D.to_device_colmajor(dst0) if beta != 0 else torch.full((batch, n), float("nan"), device="cuda:0")
        _lib.check(L.cuvdia_set_path(_lib.PATH_WALK), "set_path")
        try:
            D.prod_bias_act(dd, dev, Bd, trans, alpha, beta, bd if use_bias else None,
                            _lib.ACT_SIGMOID if act else _lib.ACT_NONE)
            assert L.cuvdia_last_path() == _lib.PATH_WALK
            assert L.cuvdia_last_kernel().decode().endswith(", true>")
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
        assert np.all(np.abs(got - ref) <= tol), (alpha, beta, use_bias, act, float((np.abs(got - ref) / tol).max()))
    # the sampled form: dst = (p > u) with u(row, column) the documented Philox draw; the oracle's bits wherever the two
    # sides' p cannot straddle u (the rule of the tile-by-tile kernel's test), for beta == 0 and beta != 0
    for seed, beta in ((0, 0.0), (0x9E3779B97F4A7C15, 0.0), (12345, 0.5)):
        p_ref = oracle.prod_bias_act(A, B, dst0 if beta != 0 else None, trans, 1.0, beta, bias, True)
        mag = oracle.prod_mag(A, B, dst0 if beta != 0 else None, trans, 1.0, beta) + np.abs(bias)[:, None]
        u = oracle.sample_uniform(n, batch, seed)
        ref = oracle.rnd_binarize(p_ref, u)
        decided = np.abs(p_ref.astype(np.float64) - u) > 0.25e-5 * mag + 4e-7
        assert decided.mean() > 0.999
        dd = D.to_device_colmajor(dst0) if beta != 0 else torch.full((batch, n), float("nan"), device="cuda:0")
        L.cuvdia_set_path(_lib.PATH_WALK)
        try:
            D.prod_bias_act(dd, dev, Bd, trans, 1.0, beta, bd, _lib.ACT_SIGMOID_SAMPLE, seed=seed)
            assert L.cuvdia_last_path() == _lib.PATH_WALK
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)
        got = D.to_host_colmajor(dd)
        assert np.all((got == 0.0) | (got == 1.0))
        assert np.array_equal(got[decided], ref[decided]), (seed, beta, int((got != ref)[decided].sum()))


@pytest.mark.parametrize("trans", ["n", "t"])
def test_walk_on_a_rectangular_matrix_with_a_short_last_segment(oracle, gu, trans):
    """60 row tiles per walk: the last segment is shorter than the others, and the window hangs over the
    operand's end in one direction only."""
    from cuv_amd import _lib
    rng = np.random.default_rng(5)
    h, w = (64 * 60, 64 * 64) if trans == "n" else (64 * 64, 64 * 60)
    A = _window_dia(oracle, rng, h, w, 64, 7)
    B, dst = _operands(rng, A, 96, trans)
    _, ran = gu.check_prod(oracle, A, B, dst, trans, 1.0, 0.5, _lib.PATH_WALK, "walk rectangular")
    assert ran == _lib.PATH_WALK


def test_walk_is_refused_where_its_shape_conditions_fail(oracle, gu):
    """A 48-wide map (window rows 48 apart: not a multiple of the tile's 64 rows) and a 9x9 window have no
    walking kernel: forcing it is an error, the automatic choice falls back to the tile-by-tile kernel."""
    from cuv_amd import _lib
    rng = np.random.default_rng(7)
    for px, fs in ((48, 7), (64, 9)):
        n = px * px
        A = _window_dia(oracle, rng, n, n, px, fs)
        B, dst = _operands(rng, A, 64, "n")
        with pytest.raises(_lib.CuvDiaError):
            gu.gpu_prod(A, B, dst, "n", 1.0, 0.0, _lib.PATH_WALK)
        _, ran = gu.check_prod(oracle, A, B, dst, "n", 1.0, 0.0, _lib.PATH_AUTO, "fallback")
        assert ran == _lib.PATH_TILED


@pytest.mark.parametrize("trans", ["n", "t"])
def test_automatic_choice_walks_a_large_product(oracle, gu, trans):
    """128x128 map, 7x7 window, batch 1536: 6144 tiles -- the automatic choice takes the walking kernel, and
    a small batch on the same matrix stays with the tile-by-tile kernel."""
    from cuv_amd import _lib
    rng = np.random.default_rng(8)
    n = 128 * 128
    A = _window_dia(oracle, rng, n, n, 128, 7)
    dev = gu.make_dev_dia(A)
    B, dst = _operands(rng, A, 1536, trans)
    _, ran = gu.check_prod(oracle, A, B, dst, trans, 1.0, 0.5, _lib.PATH_AUTO, "auto large", dev=dev)
    assert ran == _lib.PATH_WALK
    B, dst = _operands(rng, A, 128, trans)
    _, ran = gu.check_prod(oracle, A, B, dst, trans, 1.0, 0.5, _lib.PATH_AUTO, "auto small", dev=dev)
    assert ran == _lib.PATH_TILED


@pytest.mark.parametrize("trans", ["n", "t"])
def test_walk_on_column_slices_of_wider_allocations(oracle, gu, trans):
    """ld > rows for both dense operands, NaN in every gap of the input (and before its first and behind its last
    column), a sentinel in the gaps of the destination: the walking kernel's staged blocks run 6 rows past a
    tile and start up to 3 rows before it -- nothing of that may come from a gap, and nothing but the
    destination's own rows may be written.  beta != 0 also reads the destination through the view."""
    import torch
    from cuv_amd import dia as D, _lib
    rng = np.random.default_rng(11)
    px, batch = 64, 70
    n = px * px
    A = _window_dia(oracle, rng, n, n, px, 7)
    B, dst = _operands(rng, A, batch, trans)
    Ad = gu.make_dev_dia(A)
    ldb, ldd = n + 12, n + 20
    Bbig = torch.full((batch + 2, ldb), float("nan"), device="cuda:0")
    Bbig[1:batch + 1, :n] = D.to_device_colmajor(B)
    Dbig = torch.full((batch + 2, ldd), -7.0, device="cuda:0")
    Dbig[1:batch + 1, :n] = D.to_device_colmajor(dst)
    L = _lib.lib()
    L.cuvdia_set_path(_lib.PATH_WALK)
    try:
        D.prod(Dbig[1:batch + 1, :n], Ad, Bbig[1:batch + 1, :n], trans, "n", 0.75, -1.5)
        assert L.cuvdia_last_path() == _lib.PATH_WALK
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    got = D.to_host_colmajor(Dbig[1:batch + 1, :n])
    gu.assert_close_mag(got, oracle.prod(A, B, dst, trans, 0.75, -1.5), oracle.prod_mag(A, B, dst, trans, 0.75, -1.5), "walk ld view")
    assert torch.all(Dbig[:, n:] == -7.0) and torch.all(Dbig[0] == -7.0) and torch.all(Dbig[batch + 1] == -7.0)


def test_walk_under_graph_capture_and_replay(oracle, gu):
    """The walking kernel recorded into a HIP graph and replayed with the program's own eager work between the
    replays: every replay equals the eager result."""
    import torch
    from cuv_amd import dia as D, _lib
    rng = np.random.default_rng(12)
    px, batch = 64, 96
    n = px * px
    A = _window_dia(oracle, rng, n, n, px, 5)
    B, dst0 = _operands(rng, A, batch, "n")
    Ad = gu.make_dev_dia(A)
    Bd = D.to_device_colmajor(B)
    L = _lib.lib()
    L.cuvdia_set_path(_lib.PATH_WALK)
    try:
        eager = torch.zeros(batch, n, device="cuda:0")
        D.prod(eager, Ad, Bd, "n", "n", 1.0, 0.0)
        assert L.cuvdia_last_path() == _lib.PATH_WALK
        out = torch.zeros(batch, n, device="cuda:0")
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            D.prod(out, Ad, Bd, "n", "n", 1.0, 0.0, sync=False)          # warm-up on a side stream
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            D.prod(out, Ad, Bd, "n", "n", 1.0, 0.0, sync=False)          # (a synchronisation would end the capture)
        for rep in range(3):
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), "replay %d differs from the eager call" % rep
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    gu.assert_close_mag(D.to_host_colmajor(eager), oracle.prod(A, B), oracle.prod_mag(A, B), "walk eager")


@pytest.mark.parametrize("seed", range(16))
def test_walk_on_random_window_shapes(oracle, gu, seed):
    """Seeded draws of the map (width a multiple of 64, any height), window (3, 5, 7), channels, a matrix that is
    square or a few rows wider or narrower, batch and factors; both transposes, the walking kernel forced."""
    from cuv_amd import _lib
    rng = np.random.default_rng(9000 + seed)
    px = int(rng.choice([64, 128, 192, 256, 320]))
    fs = int(rng.choice([3, 5, 7]))
    ch = int(rng.choice([1, 1, 2, 3]))
    py = int(rng.integers(fs + 1, 40))
    n = px * py
    r = fs // 2
    offs = [c * n + dy * px + dx for c in range(ch) for dy in range(-r, r + 1) for dx in range(-r, r + 1)]
    h = n * ch
    w = h + int(rng.choice([0, 0, px, -px, 64])) if ch == 1 else h
    batch = int(rng.choice([1, 24, 40, 64, 65, 128, 200, 300]))
    alpha, beta = float(rng.uniform(-2, 2)), float(rng.choice([0.0, 1.0, rng.uniform(-1, 1)]))
    A = oracle.Dia(h, w, offs, None, 1)
    A.vals[:] = np.nan
    m = oracle.valid_mask(A)
    A.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    for trans in ("n", "t"):
        B, dst = _operands(rng, A, batch, trans)
        what = "seed %d: map %dx%d, window %d, %d channels, %dx%d, batch %d, '%s'" % (seed, px, py, fs, ch, h, w, batch, trans)
        print(what, flush=True)
        _, ran = gu.check_prod(oracle, A, B, None if beta == 0.0 else dst, trans, alpha, beta, _lib.PATH_WALK, what)
        assert ran == _lib.PATH_WALK


@pytest.mark.parametrize("trans", ["n", "t"])
def test_walk_non_finite_values_reach_only_the_rows_that_use_them(oracle, gu, trans):
    """Inf and NaN in B, in the interior and in the first and last rows of the operand: the walking kernel stages
    zeros for rows outside the operand and for diagonal slots outside the matrix, and no such zero may meet a
    non-finite dense value that the oracle's loop over stored elements does not touch."""
    from cuv_amd import _lib
    rng = np.random.default_rng(81)
    px, fs, batch = 64, 7, 70
    n = px * px
    A = _window_dia(oracle, rng, n, n, px, fs)
    B, _ = _operands(rng, A, batch, trans)
    B[2000, 3] = np.inf
    B[1, 40] = np.nan
    B[n - 2, 5] = -np.inf
    B[777, 69] = np.nan
    with np.errstate(invalid="ignore"):
        ref = oracle.prod(A, B, None, trans)
    got, ran = gu.gpu_prod(A, B, None, trans, 1.0, 0.0, _lib.PATH_WALK)
    assert ran == _lib.PATH_WALK
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    fin = np.isfinite(ref)
    np.testing.assert_allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-5)
