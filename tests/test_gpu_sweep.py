"""Seeded random sweep: both kernel families of the HIP path against the CPU
oracle on shapes nobody picked by hand -- ragged sizes, shuffled, duplicate and
out-of-range offsets, steep matrices (row factor 2-4), operands that are misaligned views of wider allocations
(any leading dimension, base address not a multiple of 16 bytes), beta == 0 over
NaN destinations.  The allocations around the INPUT views hold NaN, so a kernel
that lets a byte of the gap between columns (or before the first, after the
last column) reach a stored result fails.  Tolerance as in test_gpu_parity
(1e-5 of the summed magnitudes); bytes around the destination view must stay
as they were.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _offsets(rng, h, w):
    offs = []
    for _ in range(int(rng.integers(1, 6))):
        start = int(rng.integers(-h - 2, w + 2))
        step = 1 if rng.random() < 0.85 else int(rng.integers(2, 5))
        offs += [start + k * step for k in range(int(rng.integers(1, 20)))]
    if rng.random() < 0.3:
        offs += [int(x) for x in rng.integers(-h, w, int(rng.integers(1, 5)))]
    if rng.random() < 0.5:
        offs = sorted(set(offs))
    else:
        rng.shuffle(offs)
    return offs[:60]


def _view(torch, rng, host, fill=float("nan")):
    """(rows, batch) host matrix -> (flat allocation, (batch, rows) view of it with a random leading dimension
    and a base shifted by 0-3 floats, mask of the view's elements in the allocation)"""
    rows, batch = host.shape
    ld = rows + (int(rng.integers(0, 9)) if rng.random() < 0.7 else 0)
    shift = int(rng.integers(0, 4)) if rng.random() < 0.5 else 0
    flat = torch.full((batch * ld + shift + 8,), fill, device="cuda:0")
    v = flat[shift:shift + batch * ld].view(batch, ld)[:, :rows]
    v.copy_(torch.from_numpy(np.ascontiguousarray(host.T)))
    inside = torch.zeros(flat.numel(), dtype=torch.bool, device="cuda:0")
    inside[shift:shift + batch * ld].view(batch, ld)[:, :rows] = True
    return flat, v, inside


def _one_case(oracle, seed, lo, hi):
    import torch
    import _gpu_util as gu
    from cuv_amd import _lib, dia as D
    L = _lib.lib()
    rng = np.random.default_rng(seed)
    h, w = int(rng.integers(lo, hi)), int(rng.integers(lo, hi))
    if rng.random() < 0.3:
        w = h
    offs = _offsets(rng, h, w)
    batch = int(rng.choice([1, 2, 5, 23, 24, 25, 63, 64, 65, 100, 128, 130, 200]))
    alpha = float(rng.choice([1.0, -0.5, 2.25]))
    beta = float(rng.choice([0.0, 0.0, 1.0, -1.5]))
    stride = max(h, w) + (int(rng.integers(0, 7)) if rng.random() < 0.5 else 0)
    rf = int(rng.choice([2, 3, 4])) if rng.random() < 0.15 else 1        # steep matrices: the generic kernels only
    A = oracle.Dia(h, w, offs, stride, rf)
    A.vals[:] = np.nan
    valid = oracle.valid_mask(A)
    A.vals[valid] = rng.uniform(-1, 1, int(valid.sum())).astype(np.float32)
    Ad = gu.make_dev_dia(A)
    what = "seed %d: %dx%d, row factor %d, %d offsets, batch %d, alpha %g, beta %g" % (
        seed, h, w, rf, len(offs), batch, alpha, beta)

    def forced(path, call):
        """runs call() on the given kernel family; False when the tiled family does not take the shape"""
        L.cuvdia_set_path(path)
        try:
            call()
        except _lib.CuvDiaError:
            assert path == _lib.PATH_TILED, what
            return False
        finally:
            L.cuvdia_set_path(_lib.PATH_AUTO)
        return True

    for trans in ("n", "t"):
        n_in, n_out = (h, w) if trans == "t" else (w, h)
        B = np.asfortranarray(rng.uniform(-1, 1, (n_in, batch)).astype(np.float32))
        dst = np.asfortranarray(rng.uniform(-1, 1, (n_out, batch)).astype(np.float32))
        ref = oracle.prod(A, B, dst if beta != 0 else None, trans, alpha, beta)
        mag = oracle.prod_mag(A, B, dst if beta != 0 else None, trans, alpha, beta)
        for path in (_lib.PATH_GENERIC, _lib.PATH_TILED):
            _, Bv, _ = _view(torch, rng, B)
            flat, Dv, inside = _view(torch, rng, dst, fill=-7.0)
            if beta == 0:
                Dv.fill_(float("nan"))
            before = flat.clone()
            if not forced(path, lambda: D.prod(Dv, Ad, Bv, trans, "n", alpha, beta)):
                continue
            gu.assert_close_mag(D.to_host_colmajor(Dv), ref, mag, "%s, prod %s, path %d" % (what, trans, path))
            assert torch.equal(flat[~inside], before[~inside]), what + ": wrote outside the destination view"

    P = np.asfortranarray(rng.uniform(-1, 1, (h, batch)).astype(np.float32))
    Q = np.asfortranarray(rng.uniform(-1, 1, (w, batch)).astype(np.float32))
    C = oracle.Dia(h, w, offs, stride, rf, A.vals.copy())
    if beta == 0:
        C.vals[valid] = np.nan
    ref = oracle.dd2dia(C, P, Q, alpha, beta)
    mag = oracle.dd2dia_f64(oracle.Dia(h, w, offs, stride, rf, np.abs(np.nan_to_num(C.vals))),
                            np.abs(P), np.abs(Q), abs(alpha), abs(beta))
    for path in (_lib.PATH_GENERIC, _lib.PATH_TILED):
        Cd = gu.make_dev_dia(C)
        _, Pv, _ = _view(torch, rng, P)
        _, Qv, _ = _view(torch, rng, Q)
        if not forced(path, lambda: D.densedense_to_dia(Cd, None, Pv, Qv, alpha, beta)):
            continue
        got = Cd.pull()
        assert np.array_equal(got[~valid].view(np.uint32), C.vals[~valid].view(np.uint32)), what + ": padding written"
        gu.assert_close_mag(got[valid], ref[valid], mag[valid], "%s, projection, path %d" % (what, path))


@pytest.mark.parametrize("first", range(0, 120, 20))
def test_small_shapes(oracle, first):
    for seed in range(first, first + 20):
        _one_case(oracle, seed, 1, 300)


@pytest.mark.parametrize("first", range(1000, 1060, 10))
def test_shapes_of_many_tiles(oracle, first):
    for seed in range(first, first + 10):
        _one_case(oracle, seed, 900, 6000)
