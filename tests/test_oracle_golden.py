"""Pins the CPU oracle without running the reference.

Three kinds of evidence, chosen so that a dropped term, a wrong sign, a
shifted index or a transposed operand fails at least one:
  * the exact-integer closed forms of the reference's own sequence() fixtures
    (tests/golden/*.json; src/tests/spmv.cpp, densedense_to_dia.cpp,
    dia_mat.cpp, convert.cpp),
  * reduction to textbook routines: DIA product == dense fp64 GEMM of the
    densified matrix, 't' == product with the explicit transpose, dd2dia ==
    band projection of a brute-force A*B',
  * invariants: linearity in alpha, beta == 0 never reads dst, padding slots
    untouched, adjoint identity <A*V, H> == <proj(H*V'), A>.
"""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


def _seq_dia(o, fx):
    d = o.Dia(fx["h"], fx["w"], fx["offsets"], fx["stride"], fx["rf"])
    d.vals[:] = np.arange(d.vals.size, dtype=np.float32)
    return d


def _seq(rows, cols):
    return np.arange(rows * cols, dtype=np.float32).reshape(cols, rows).T.copy(order="F")


# ---------------------------------------------------------------- golden ---
def test_spmv_fixture_plain(oracle):
    fx = _load("spmv_fixture.json")
    A = _seq_dia(oracle, fx)
    B = _seq(fx["w"], fx["batch"])
    C = _seq(fx["h"], fx["batch"])
    got = oracle.prod(A, B, None, "n", 1.0, 0.0)
    assert np.array_equal(got, np.asarray(fx["AB"], np.float32))
    got_t = oracle.prod(A, C, None, "t", 1.0, 0.0)
    assert np.array_equal(got_t, np.asarray(fx["AtC"], np.float32))


def test_spmv_fixture_scaled(oracle):
    # spmv.cpp:116-143 -- factAv = 2, factC = 1.3 on a sequence()-filled dst
    fx = _load("spmv_fixture.json")
    A = _seq_dia(oracle, fx)
    B = _seq(fx["w"], fx["batch"])
    C = _seq(fx["h"], fx["batch"])
    got = oracle.prod(A, B, C, "n", 2.0, 1.3)
    np.testing.assert_allclose(got, np.asarray(fx["n_alpha2_beta1p3"]), rtol=2e-6)
    got_t = oracle.prod(A, C, B, "t", 2.0, 1.3)
    np.testing.assert_allclose(got_t, np.asarray(fx["t_alpha2_beta1p3"]), rtol=2e-6)


def test_dd2dia_fixture(oracle):
    # densedense_to_dia.cpp:109-164 -- rf = 4, C.vec() zeroed, defaults (1, 0)
    fx = _load("dd2dia_fixture.json")
    C = oracle.Dia(fx["h"], fx["w"], fx["offsets"], fx["stride"], fx["rf"])
    A = _seq(fx["h"], fx["batch"])
    B = _seq(fx["w"], fx["batch"])
    exp = np.asarray([[np.nan if v is None else v for v in row] for row in fx["expected"]],
                     np.float64).reshape(-1)
    valid = ~np.isnan(exp)
    assert np.array_equal(valid, oracle.valid_mask(C))
    for got in (oracle.dd2dia_literal(C, A, B), oracle.dd2dia(C, A, B, 1.0, 0.0),
                oracle.dd2dia(C, A, B, 1.0, 1.0)):
        assert np.array_equal(got[valid].astype(np.float64), exp[valid])
        assert np.all(got[~valid] == 0)


def test_dia_dense_fixture(oracle):
    for fx in _load("dia_dense_fixture.json"):
        A = _seq_dia(oracle, fx)
        exp = np.asarray(fx["dense"], np.float32)
        assert np.array_equal(oracle.to_dense(A), exp)
        for i in range(fx["h"]):
            for j in range(fx["w"]):
                assert oracle.get(A, i, j) == exp[i, j]


# ------------------------------------------------- textbook cross-checks ---
def _rand_dia(o, rng, h, w, offsets, rf=1, stride=None, pad=np.nan):
    d = o.Dia(h, w, offsets, stride, rf)
    d.vals[:] = pad                     # padding the host loops must never read
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    return d


def _dense64(o, d):
    """Densify by the addressing rule alone (independent of to_dense)."""
    M = np.zeros((d.h, d.w))
    for di, k in enumerate(d.offsets.tolist()):
        for i in range(d.h):
            j = k + i // d.rf
            if 0 <= j < d.w:
                M[i, j] += float(d.vals[di * d.stride + i])
    return M


CASES = [
    (32, 16, [-3, -2, -1, 0, 1, 2, 3], 1),
    (16, 32, [0, 1, -1], 1),                   # unsorted table, wide
    (40, 40, [5, -7, 0, 39, -39], 1),          # corner diagonals
    (36, 19, [-3, -2, -1, 0, 1, 2, 3], 4),     # steep
    (24, 12, [2, -1, 0, 4], 2),
    (20, 20, [0], 1),                          # one diagonal: element-wise product
    (12, 30, [-11, 29, 3], 1),
]


@pytest.mark.parametrize("h,w,offs,rf", CASES)
@pytest.mark.parametrize("trans", ["n", "t"])
def test_prod_equals_dense_gemm(oracle, h, w, offs, rf, trans):
    rng = np.random.default_rng(h * 131 + w)
    d = _rand_dia(oracle, rng, h, w, offs, rf)
    M = _dense64(oracle, d)
    n_in = h if trans == "t" else w
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, 5)).astype(np.float32))
    ref = (M.T if trans == "t" else M) @ B.astype(np.float64)
    got = oracle.prod(d, B, None, trans)
    mag = oracle.prod_mag(d, B, None, trans)
    assert np.all(np.abs(got - ref) <= 4e-7 * len(offs) * rf * np.maximum(mag, 1e-30) + 1e-30)
    np.testing.assert_allclose(oracle.prod_f64(d, B, None, trans), ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(mag, np.abs(M.T if trans == "t" else M) @ np.abs(B).astype(np.float64),
                               rtol=1e-12)
    # densify via the reference's convert loop agrees with the addressing rule
    assert np.array_equal(oracle.to_dense(d).astype(np.float64), M)


def test_single_main_diagonal_is_elementwise(oracle):
    rng = np.random.default_rng(3)
    d = _rand_dia(oracle, rng, 20, 20, [0])
    x = rng.uniform(-1, 1, 20).astype(np.float32)
    assert np.array_equal(oracle.spmv(d, x, np.zeros(20, np.float32)), d.vals[:20] * x)


def _identity_dia(o, n):
    d = o.Dia(n, n, [0], None, 1)
    d.vals[:] = 0
    d.vals[:n] = 1
    return d


def test_bias_act_on_identity_is_the_logistic_function(oracle):
    """With A the identity the layer update is sigmoid(x + bias) element by element: checked against
    1 / (1 + exp(-t)) evaluated in fp64 by math.exp on the fp32 sum t, to fp32 rounding of the steps
    (expf, the add, the divide: below 1e-7 absolute on values in (0, 1))."""
    import math
    n, batch = 37, 5
    rng = np.random.default_rng(31)
    d = _identity_dia(oracle, n)
    X = np.asfortranarray(rng.uniform(-6, 6, (n, batch)).astype(np.float32))
    bias = rng.uniform(-2, 2, n).astype(np.float32)
    got = oracle.prod_bias_act(d, X, None, "n", 1.0, 0.0, bias=bias, sigmoid=True)
    assert got.dtype == np.float32 and got.shape == (n, batch)
    worst = 0.0
    for i in range(n):
        for j in range(batch):
            t = float(np.float32(X[i, j] + bias[i]))
            worst = max(worst, abs(float(got[i, j]) - 1.0 / (1.0 + math.exp(-t))))
    assert worst <= 1e-7, worst
    # the transposed product of the identity is the same update
    assert np.array_equal(got, oracle.prod_bias_act(d, X, None, "t", 1.0, 0.0, bias=bias, sigmoid=True))
    # without the activation: the sum itself, rounded once
    lin = oracle.prod_bias_act(d, X, None, "n", 1.0, 0.0, bias=bias, sigmoid=False)
    assert np.array_equal(lin, (X + bias[:, None]).astype(np.float32))


def test_bias_act_bias_is_added_per_row_and_exactly(oracle):
    """The bias belongs to the output ROW (matrix_plus_col) and enters after the product: with power-of-two
    biases and small-integer operands every step is exact, so the difference of two runs is the bias itself --
    a bias added per column, before alpha, or scaled by beta fails."""
    rng = np.random.default_rng(32)
    h, w, batch = 24, 30, 6
    d = _rand_dia(oracle, rng, h, w, [-3, 0, 2, 9])
    d.vals[:] = np.where(np.isnan(d.vals), d.vals, np.round(d.vals * 4))
    B = np.asfortranarray(rng.integers(-3, 4, (w, batch)).astype(np.float32))
    dst = np.asfortranarray(rng.integers(-3, 4, (h, batch)).astype(np.float32))
    bias = (2.0 ** rng.integers(-2, 4, h)).astype(np.float32)
    base = oracle.prod_bias_act(d, B, dst, "n", 2.0, -0.5, bias=None, sigmoid=False)
    withb = oracle.prod_bias_act(d, B, dst, "n", 2.0, -0.5, bias=bias, sigmoid=False)
    assert np.array_equal(base, oracle.prod(d, B, dst, "n", 2.0, -0.5))
    assert np.array_equal(withb - base, np.broadcast_to(bias[:, None], (h, batch)))
    # transposed: the bias has one entry per column of A
    bias_t = (2.0 ** rng.integers(-2, 4, w)).astype(np.float32)
    Bt = np.asfortranarray(rng.integers(-3, 4, (h, batch)).astype(np.float32))
    base_t = oracle.prod_bias_act(d, Bt, None, "t", 1.0, 0.0)
    with_t = oracle.prod_bias_act(d, Bt, None, "t", 1.0, 0.0, bias=bias_t)
    assert np.array_equal(with_t - base_t, np.broadcast_to(bias_t[:, None], (w, batch)))


def test_bias_act_special_values(oracle):
    """sigmoid(0) == 0.5 exactly; large arguments saturate to 0 and 1 without NaN; sigmoid(-t) == 1 - sigmoid(t)
    to one rounding."""
    n = 8
    d = _identity_dia(oracle, n)
    X = np.zeros((n, 3), np.float32, order="F")
    assert np.array_equal(oracle.prod_bias_act(d, X, sigmoid=True), np.full((n, 3), 0.5, np.float32))
    # a bias cancelling the input lands on 0.5 too
    X[:] = 1.25
    got = oracle.prod_bias_act(d, X, bias=np.full(n, -1.25, np.float32), sigmoid=True)
    assert np.array_equal(got, np.full((n, 3), 0.5, np.float32))
    with np.errstate(over="ignore"):
        X[:, 0], X[:, 1], X[:, 2] = 200.0, -200.0, 3.0
        sat = oracle.prod_bias_act(d, X, sigmoid=True)
        assert np.all(sat[:, 0] == 1.0) and np.all(sat[:, 1] == 0.0) and not np.isnan(sat).any()
        X[:, 1] = -3.0
        sym = oracle.prod_bias_act(d, X, sigmoid=True)
    assert np.all(np.abs(sym[:, 1] - (np.float32(1) - sym[:, 2])) <= 6e-8)


def test_trans_equals_explicit_transpose(oracle):
    rng = np.random.default_rng(4)
    h, w, offs = 30, 22, [-4, 0, 1, 7]
    d = _rand_dia(oracle, rng, h, w, offs)
    # A^T stored as its own DIA matrix: offsets negate, slot index becomes column
    t = oracle.Dia(w, h, [-k for k in offs], max(h, w), 1)
    for di, k in enumerate(offs):
        for i in range(h):
            j = i + k
            if 0 <= j < w:
                t.vals[di * t.stride + j] = d.vals[di * d.stride + i]
    X = np.asfortranarray(rng.uniform(-1, 1, (h, 3)).astype(np.float32))
    a = oracle.prod(d, X, None, "t")
    b = oracle.prod(t, X, None, "n")
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-6)


def test_beta_zero_never_reads_dst_and_scaling(oracle):
    rng = np.random.default_rng(5)
    d = _rand_dia(oracle, rng, 32, 16, [-3, -2, -1, 0, 1, 2, 3])
    B = np.asfortranarray(rng.uniform(-1, 1, (16, 4)).astype(np.float32))
    nan_dst = np.full((32, 4), np.nan, np.float32, order="F")
    y0 = oracle.prod(d, B, nan_dst, "n", 1.0, 0.0)
    assert np.isfinite(y0).all()
    y2 = oracle.prod(d, B, nan_dst, "n", 2.0, 0.0)       # power-of-two alpha: exact
    assert np.array_equal(y2, 2 * y0)
    dst = np.asfortranarray(rng.uniform(-1, 1, (32, 4)).astype(np.float32))
    y = oracle.prod(d, B, dst, "n", 1.0, 0.5)
    np.testing.assert_allclose(y, 0.5 * dst + y0, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("h,w,offs,rf", [c for c in CASES if c[0] % c[3] == 0])
def test_dd2dia_equals_projected_outer_product(oracle, h, w, offs, rf):
    rng = np.random.default_rng(h * 7 + w)
    batch = 9
    C = _rand_dia(oracle, rng, h, w, offs, rf, pad=-77.0)
    A = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    B = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    full = A.astype(np.float64) @ B.astype(np.float64).T          # brute force A*B'
    valid = oracle.valid_mask(C)
    exp = C.vals.astype(np.float64).copy()
    alpha, beta = 0.25, 0.9
    for di, k in enumerate(offs):
        for i in range(h):
            j = k + i // rf
            if 0 <= j < w:
                s = di * C.stride + i
                exp[s] = np.float64(np.float32(beta)) * exp[s] + np.float64(np.float32(alpha)) * full[i, j]
    got = oracle.dd2dia(C, A, B, alpha, beta)
    np.testing.assert_allclose(got[valid], exp[valid], rtol=2e-6, atol=2e-6)
    assert np.all(got[~valid] == np.float32(-77.0))               # padding untouched
    np.testing.assert_allclose(oracle.dd2dia_f64(C, A, B, alpha, beta)[valid], exp[valid],
                               rtol=1e-12, atol=1e-12)
    # the literal host loop is the alpha = beta = 1 case
    lit = oracle.dd2dia_literal(C, A, B)
    np.testing.assert_allclose(lit[valid], oracle.dd2dia(C, A, B, 1.0, 1.0)[valid], rtol=2e-6, atol=2e-6)
    # beta == 0 ignores what dst held
    Cn = oracle.Dia(h, w, offs, C.stride, rf, np.full_like(C.vals, np.nan))
    z = oracle.dd2dia(Cn, A, B, 1.0, 0.0)
    assert np.isfinite(z[valid]).all() and np.isnan(z[~valid]).all()
    # linear in a power-of-two alpha
    assert np.array_equal(oracle.dd2dia(Cn, A, B, 4.0, 0.0)[valid], 4 * z[valid])


def test_adjoint_identity(oracle):
    """<A*V, H> == <proj(H*V'), A>: ties the SpMM and the projected outer
    product together (an index slip in either breaks it)."""
    rng = np.random.default_rng(11)
    h, w, offs, b = 48, 40, [-9, -1, 0, 2, 17], 6
    A = _rand_dia(oracle, rng, h, w, offs, pad=0.0)
    V = np.asfortranarray(rng.uniform(-1, 1, (w, b)).astype(np.float32))
    H = np.asfortranarray(rng.uniform(-1, 1, (h, b)).astype(np.float32))
    lhs = float(np.sum(oracle.prod_f64(A, V, None, "n") * H))
    G = oracle.Dia(h, w, offs, A.stride, 1)
    g = oracle.dd2dia_f64(G, H, V, 1.0, 0.0)
    rhs = float(np.sum(g * A.vals.astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-10 * max(1.0, abs(lhs))
    # and the transposed product is the adjoint of the normal one
    lhs_t = float(np.sum(oracle.prod_f64(A, H, None, "t") * V))
    assert abs(lhs - lhs_t) <= 1e-10 * max(1.0, abs(lhs))


def test_out_of_range_and_duplicate_offsets(oracle):
    rng = np.random.default_rng(12)
    # offsets outside the matrix contribute nothing; duplicates both contribute
    d = _rand_dia(oracle, rng, 10, 10, [0, 0, 25, -25, 3], pad=0.0)
    x = rng.uniform(-1, 1, 10).astype(np.float32)
    M = _dense64(oracle, d)
    np.testing.assert_allclose(oracle.spmv(d, x, np.zeros(10, np.float32)), M @ x, rtol=1e-5, atol=1e-6)
    # element access: the last table entry with an offset wins
    assert oracle.get(d, 2, 2) == d.vals[1 * d.stride + 2]


def test_rf_not_dividing_is_rejected_by_literal_loop(oracle):
    C = oracle.Dia(10, 6, [0, 1], 10, 4)
    A = np.ones((10, 2), np.float32, order="F")
    B = np.ones((6, 2), np.float32, order="F")
    with pytest.raises(RuntimeError):
        oracle.dd2dia_literal(C, A, B)


# ------------------------------------------------------ next-row helpers ---
def test_filter_offsets_closed_form(oracle):
    # filter_factory.hpp:43-76 with one map in and out: the centred window
    offs = oracle.filter_offsets(128, 128, 7, 1, 1)
    exp = [dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    assert offs.tolist() == exp
    offs = oracle.filter_offsets(8, 8, 3, 2, 3)
    exp = [(m - 1) * 64 + (i - 1) * 8 + (j - 1) for m in range(4) for i in range(3) for j in range(3)]
    assert offs.tolist() == exp


def test_avg_diagonals_closed_form(oracle):
    fx = _load("dia_dense_fixture.json")[0]
    A = _seq_dia(oracle, fx)
    got = oracle.avg_diagonals(A)
    exp = []
    for d, k in enumerate(fx["offsets"]):
        i0, j0 = max(0, -k), max(0, k)
        n = min(fx["h"] - i0, fx["w"] - j0)
        exp.append(sum(fx["stride"] * d + i for i in range(i0, i0 + n)) / n)
    np.testing.assert_allclose(got, exp, rtol=1e-6)


# ------------------------------------------------------------ workloads ---
def test_workload_counts_match_published_table():
    from cuv_amd import workloads as W
    assert W.pattern_cfg0().nnz == 134896
    p = W.pattern_lc7()
    assert p.nd == 49 and p.nnz == 792052
    assert W.spmm_bytes(p, 128, "n", 0.0) == 19945620
    assert W.spmm_bytes(p, 128, "t", 0.5) == 28334228
    assert W.dd2dia_bytes(p, 128, 0.9) == 23113828
    assert W.flops(p, 128) == 202765312
    q = W.pattern_large()
    assert q.nd == 676 and q.nnz == 110616022
    assert W.spmm_bytes(q, 256, "n", 0.0) == 979337704


# ----------------------------------------------------------- Philox sampling ---
def test_philox_known_answers(oracle):
    """Random123's published known-answer vectors for philox4x32-10 (kat_vectors:
    counter, key -> output)."""
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        got = oracle.philox4x32_10(np.array(ctr, np.uint32), np.array(key, np.uint32))
        assert [int(x) for x in got] == list(want)


def test_sample_uniform_indexing(oracle):
    """u(row, col) takes word col & 3 of the block at counter (row, col >> 2, 0, 0)
    -- checked element by element against single-block calls -- lies in [0, 1),
    is a multiple of 2^-24 and is uniform enough for a 4-sigma test."""
    seed = 0x0123456789ABCDEF
    u = oracle.sample_uniform(9, 11, seed)
    key = np.array([seed & 0xFFFFFFFF, seed >> 32], np.uint32)
    for r in range(9):
        for c in range(11):
            blk = oracle.philox4x32_10(np.array([r, c >> 2, 0, 0], np.uint32), key)
            assert u[r, c] == np.float32(int(blk[c & 3]) >> 8) * np.float32(2.0 ** -24)
    big = oracle.sample_uniform(256, 256, 42)
    assert big.min() >= 0.0 and big.max() < 1.0
    assert np.all(big * 2 ** 24 == np.round(big * 2 ** 24))
    assert abs(float(big.mean()) - 0.5) < 4 * (1 / np.sqrt(12)) / 256
    assert np.array_equal(oracle.rnd_binarize(np.array([[0.5, 0.5]]), np.array([[0.25, 0.5]])), [[1.0, 0.0]])


def test_learn_step_weight_decay_closed_form(oracle):
    """rprop.cu:345: alpha = -learnrate, beta = 1 - learnrate*decay.  With
    learnrate 0.5, decay 0.25, W = 8 i, dW = 2 i every product is exact:
    W' = -i + 0.875 * 8 i = 6 i."""
    i = np.arange(1000, dtype=np.float32)
    got = oracle.learn_step_weight_decay(8 * i, 2 * i, 0.5, 0.25)
    assert got.dtype == np.float32 and np.array_equal(got, 6 * i)
    assert np.array_equal(oracle.learn_step_weight_decay(i, i, 0.0, 3.0), i)


def test_learn_step_weight_decay_momentum_pins(oracle):
    """Three checks of the momentum step (rprop.cu:158-170).
    Exact arithmetic: lr 0.5, momentum weight 0.5, decay 0.25, W = 8 i, m = 4 i, dW = 2 i give
    m' = 2 i - 0.5*(2 i + 2 i) = 0 and W' = W; with dW = 0 instead m' = 2 i - i = i, W' = 9 i.
    Reduction: without momentum the step is learn_step_weight_decay (rprop.cu:341-346), whose decay shrinks
    the weights -- the sign the host loop at rprop.cu:364 gets wrong.
    The reference's own test (src/tests/optimize.cpp:89-123): 1000 steps on f(W) = 2 (W - optimum)^2 with
    learnrate 0.01 and momentum weight 1 - iter/1000 end within 0.01% of the optimum."""
    i = np.arange(1000, dtype=np.float32)
    W, m = oracle.learn_step_weight_decay_momentum(8 * i, 4 * i, 2 * i, 0.5, 0.5, 0.25)
    assert np.array_equal(W, 8 * i) and np.array_equal(m, 0 * i)
    W, m = oracle.learn_step_weight_decay_momentum(8 * i, 4 * i, 0 * i, 0.5, 0.5, 0.25)
    assert np.array_equal(W, 9 * i) and np.array_equal(m, i)

    rng = np.random.default_rng(5)
    W0 = rng.normal(0, 1, 4096).astype(np.float32)
    dW = rng.normal(0, 1, 4096).astype(np.float32)
    W, m = oracle.learn_step_weight_decay_momentum(W0, np.zeros_like(W0), dW, 0.05, 0.0, 0.002)
    plain = oracle.learn_step_weight_decay(W0, dW, 0.05, 0.002)
    assert np.allclose(W, plain, rtol=0, atol=4e-7 * (np.abs(W0) + 0.05 * np.abs(dW)).max())
    assert np.array_equal(m, (W - W0).astype(np.float32)) or np.allclose(m, W - W0, rtol=0, atol=2e-7)

    optimum = rng.random(100).astype(np.float32)
    W = rng.random(100).astype(np.float32)
    mom = np.zeros(100, np.float32)
    for it in range(1000):
        W, mom = oracle.learn_step_weight_decay_momentum(W, mom, (W - optimum).astype(np.float32), 0.01,
                                                         1.0 - it / 1000.0, 0.0)
    assert np.all(np.abs((W + 1) - (optimum + 1)) <= 1e-4 * (optimum + 1))
    assert abs(float(np.mean(2 * (W - optimum) ** 2))) <= 1e-4
