"""The rows-along-lanes SpMM kernel against the CPU oracle (forced path)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import _gpu_util
    return _gpu_util


def _window_dia(o, rng, h, w, px, fs, channels=1, map_elems=None):
    from cuv_amd import workloads as W
    d = o.Dia(h, w, W.window_offsets(px, fs, channels, map_elems), None, 1)
    d.vals[:] = np.nan
    m = o.valid_mask(d)
    d.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    return d


def _operands(rng, A, batch, trans):
    n_in, n_out = (A.h, A.w) if trans == "t" else (A.w, A.h)
    B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
    dst = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
    return B, dst


CASES = [
    # h, w, px, window, channels, batch
    (4096, 4096, 64, 7, 1, 32),
    (4096, 4096, 64, 7, 1, 70),
    (5000, 5000, 50, 7, 1, 33),
    (3000, 4100, 64, 7, 1, 40),
    (4100, 3000, 64, 7, 1, 40),
    (4096, 4096, 64, 13, 1, 64),
    (6000, 6000, 40, 13, 2, 20),
    (700, 700, 20, 7, 1, 36),
    (300, 300, 16, 13, 1, 32),
]


@pytest.mark.parametrize("h,w,px,fs,channels,batch", CASES)
@pytest.mark.parametrize("trans", ["n", "t"])
def test_rows_matches_the_oracle(oracle, gu, h, w, px, fs, channels, batch, trans):
    from cuv_amd import _lib
    rng = np.random.default_rng(h + 7 * w + px * 100 + fs * 10 + channels + batch)
    A = _window_dia(oracle, rng, h, w, px, fs, channels, map_elems=(h // channels) if channels > 1 else None)
    B, dst = _operands(rng, A, batch, trans)
    print("case", h, w, px, fs, channels, batch, trans, flush=True)
    _, ran = gu.check_prod(oracle, A, B, None, trans, 1.0, 0.0, _lib.PATH_ROWS, "rows beta0")
    assert ran == _lib.PATH_ROWS
    _, ran = gu.check_prod(oracle, A, B, dst, trans, 0.75, -1.5, _lib.PATH_ROWS, "rows scaled")
    assert ran == _lib.PATH_ROWS


@pytest.mark.parametrize("trans", ["n", "t"])
def test_rows_non_finite_values_reach_only_the_rows_that_use_them(oracle, gu, trans):
    """Inf and NaN in B, in the interior and in the first and last rows of the operand (the chunks there are
    fetched element by element, with zeros where a row does not exist): the masks of NaN and +-Inf equal the
    oracle's."""
    from cuv_amd import _lib
    rng = np.random.default_rng(82)
    h = w = 5000
    A = _window_dia(oracle, rng, h, w, 50, 7)
    B, _ = _operands(rng, A, 33, trans)
    B[2000, 3] = np.inf
    B[1, 20] = np.nan
    B[h - 2, 5] = -np.inf
    B[777, 32] = np.nan
    with np.errstate(invalid="ignore"):
        ref = oracle.prod(A, B, None, trans)
    got, ran = gu.gpu_prod(A, B, None, trans, 1.0, 0.0, _lib.PATH_ROWS)
    assert ran == _lib.PATH_ROWS
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    fin = np.isfinite(ref)
    np.testing.assert_allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-5)
