"""GPU parity on seeded random offset tables: shapes nobody chose by hand.  Every seed draws a table of one of
four kinds (scattered offsets; a few runs of consecutive offsets; a 2-d window on a px x py map, possibly with
several channels; a window plus scattered, duplicate and out-of-range offsets), a matrix size, a batch and the two
factors, and compares both products and the projection against the oracle -- automatic path and generic kernels --
with the tolerance of test_gpu_parity.py (relative 1e-5 against the magnitude sum and in the max norm)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import _gpu_util
    return _gpu_util


def _draw(seed):
    rng = np.random.default_rng(0xD1A + seed)
    kind = seed % 4
    if kind == 0:
        h, w = int(rng.integers(1, 2500)), int(rng.integers(4, 2500))
        nd = int(rng.integers(1, 30))
        offs = rng.choice(np.arange(-h + 1, w), size=min(nd, h + w - 1), replace=False).tolist()
    elif kind == 1:
        h, w = int(rng.integers(40, 3000)), int(rng.integers(40, 3000))
        offs = []
        for _ in range(int(rng.integers(1, 6))):
            start = int(rng.integers(-h + 1, w - 1))
            offs += list(range(start, min(w, start + int(rng.integers(1, 22)))))
        offs = list(dict.fromkeys(offs))                       # runs may overlap: keep the first mention
    elif kind == 2:
        px, py = int(rng.integers(8, 140)), int(rng.integers(8, 40))
        fs = int(rng.choice([3, 5, 7, 9, 13]))
        ch = int(rng.choice([1, 1, 2, 3]))
        n = px * py
        r = fs // 2
        offs = [c * n + dy * px + dx for c in range(ch) for dy in range(-r, r + 1) for dx in range(-r, r + 1)]
        h = w = n * ch
    else:
        px = int(rng.choice([16, 64, 100, 128, 256]))
        n = px * int(rng.integers(4, 24))
        h, w = n, n + int(rng.integers(0, 3)) * px
        r = int(rng.choice([1, 2, 3]))
        offs = [dy * px + dx for dy in range(-r, r + 1) for dx in range(-r, r + 1)]
        offs += rng.integers(-h + 1, w, size=int(rng.integers(0, 6))).tolist()
        offs += [w + 5, -h - 7][: int(rng.integers(0, 3))]    # outside the matrix: empty diagonals
        offs = list(dict.fromkeys(offs))
        rng.shuffle(offs)
    batch = int(rng.choice([1, 3, 24, 40, 64, 72, 128, 200, 257]))
    alpha, beta = float(rng.uniform(-2, 2)), float(rng.choice([0.0, 1.0, rng.uniform(-1, 1)]))
    return rng, h, w, [int(o) for o in offs], batch, alpha, beta


@pytest.mark.parametrize("seed", range(40))
def test_random_table(oracle, gu, seed):
    from cuv_amd import _lib
    rng, h, w, offs, batch, alpha, beta = _draw(seed)
    what = "seed %d: %dx%d, %d diagonals, batch %d" % (seed, h, w, len(offs), batch)
    print(what, flush=True)
    A = oracle.Dia(h, w, offs, None, 1)
    A.vals[:] = np.nan                                          # NaN in every padding slot
    m = oracle.valid_mask(A)
    A.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    for trans in ("n", "t"):
        n_in, n_out = (h, w) if trans == "t" else (w, h)
        B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
        dst = None if beta == 0.0 else np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
        for path in (_lib.PATH_AUTO, _lib.PATH_GENERIC):
            gu.check_prod(oracle, A, B, dst, trans, alpha, beta, path, "%s, '%s', path %d" % (what, trans, path))
    P = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    Q = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    for path in (_lib.PATH_AUTO, _lib.PATH_GENERIC):
        C = oracle.Dia(h, w, offs, A.stride, 1, A.vals.copy() if beta != 0.0 else np.full_like(A.vals, np.nan))
        gu.check_dd2dia(oracle, C, P, Q, alpha / batch, beta, path, "%s, projection, path %d" % (what, path))


@pytest.mark.parametrize("seed", range(24))
def test_random_table_non_finite(oracle, gu, seed):
    """The same tables with a handful of Inf and NaN scattered over the dense operand: the masks of NaN, +Inf and
    -Inf in both products equal the oracle's (whose loop multiplies exactly the stored elements) on the automatic
    path and on the generic kernels, and the finite results agree as in the test above."""
    from cuv_amd import _lib
    rng, h, w, offs, batch, alpha, beta = _draw(seed)
    if abs(alpha) < 1e-3:
        alpha = 1.0
    what = "seed %d: %dx%d, %d diagonals, batch %d" % (seed, h, w, len(offs), batch)
    print(what, flush=True)
    A = oracle.Dia(h, w, offs, None, 1)
    A.vals[:] = np.nan
    m = oracle.valid_mask(A)
    A.vals[m] = rng.uniform(-1, 1, int(m.sum())).astype(np.float32)
    for trans in ("n", "t"):
        n_in, n_out = (h, w) if trans == "t" else (w, h)
        B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
        for _ in range(6):
            B[int(rng.integers(0, n_in)), int(rng.integers(0, batch))] = rng.choice([np.inf, -np.inf, np.nan])
        B[0, 0], B[n_in - 1, batch - 1] = np.inf, np.nan          # the operand's corners
        dst = None if beta == 0.0 else np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
        with np.errstate(invalid="ignore"):
            ref = oracle.prod(A, B, dst, trans, alpha, beta)
        fin = np.isfinite(ref)
        with np.errstate(invalid="ignore"):
            mag = oracle.prod_mag(A, B, dst, trans, alpha, beta)
        for path in (_lib.PATH_AUTO, _lib.PATH_GENERIC):
            got, _ = gu.gpu_prod(A, B, dst, trans, alpha, beta, path)
            tag = "%s, '%s', path %d" % (what, trans, path)
            assert np.array_equal(np.isnan(got), np.isnan(ref)), tag
            assert np.array_equal(np.isposinf(got), np.isposinf(ref)), tag
            assert np.array_equal(np.isneginf(got), np.isneginf(ref)), tag
            gu.assert_close_mag(got[fin], ref[fin], mag[fin], tag)
