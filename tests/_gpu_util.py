"""Helpers shared by the GPU parity tests: run the C ABI on numpy operands and
compare against the oracle with the tolerance the tests state."""
import ctypes

import numpy as np
import torch

from cuv_amd import _lib, dia as D

REL_TOL = 1e-5          # the fp32 parity bar


def make_dev_dia(o_dia, device="cuda:0"):
    m = D.dev_dia_matrix_f(o_dia.h, o_dia.w, o_dia.nd, o_dia.stride, o_dia.rf, device=device)
    m.set_offsets(o_dia.offsets)
    m.push(o_dia.vals)
    return m


def gpu_prod(o_dia, B, dst=None, trans="n", alpha=1.0, beta=0.0, path=_lib.PATH_AUTO, dev=None):
    """Returns (result as Fortran (rows, batch) array, path that ran)."""
    L = _lib.lib()
    A = dev if dev is not None else make_dev_dia(o_dia)
    n_out = o_dia.w if trans == "t" else o_dia.h
    Bd = D.to_device_colmajor(B)
    batch = Bd.shape[0]
    if dst is None:
        dd = torch.full((batch, n_out), float("nan"), dtype=torch.float32, device="cuda:0")
    else:
        dd = D.to_device_colmajor(dst)
    _lib.check(L.cuvdia_set_path(path), "set_path")
    try:
        D.prod(dd, A, Bd, trans, "n", alpha, beta)
        ran = L.cuvdia_last_path()
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    return D.to_host_colmajor(dd), ran


def gpu_dd2dia(o_dia, A, B, alpha=1.0, beta=0.0, path=_lib.PATH_AUTO):
    L = _lib.lib()
    C = make_dev_dia(o_dia)
    Ad, Bd = D.to_device_colmajor(A), D.to_device_colmajor(B)
    bd = D.dev_block_descriptor_f(C)
    _lib.check(L.cuvdia_set_path(path), "set_path")
    try:
        D.densedense_to_dia(C, bd, Ad, Bd, alpha, beta)
        ran = L.cuvdia_last_path()
    finally:
        L.cuvdia_set_path(_lib.PATH_AUTO)
    return C.pull(), ran


def assert_close_mag(got, ref, mag, what, tol=REL_TOL):
    """|got - ref| <= tol * mag element-wise, where mag = sum of |terms| of the
    element (>= |ref|): relative 1e-5 against the scale the element was
    summed at, which stays meaningful when terms cancel.  Also demands the
    max-norm relative error stays under tol."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    mag = np.asarray(mag, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), "%s: non-finite values in GPU result" % what
    err = np.abs(got - ref)
    bad = err > tol * mag + 1e-37
    assert not bad.any(), "%s: %d elements off, worst err/mag = %.3g" % (
        what, int(bad.sum()), float((err / np.maximum(mag, 1e-37)).max()))
    scale = np.abs(ref).max()
    if scale > 0:
        assert err.max() <= tol * scale, "%s: max-norm relative error %.3g" % (what, err.max() / scale)


def check_prod(oracle, o_dia, B, dst, trans, alpha, beta, path, what, dev=None):
    got, ran = gpu_prod(o_dia, B, dst, trans, alpha, beta, path, dev=dev)
    ref = oracle.prod(o_dia, B, dst, trans, alpha, beta)
    mag = oracle.prod_mag(o_dia, B, dst, trans, alpha, beta)
    assert_close_mag(got, ref, mag, what)
    # both implementations must sit within rounding of the exact result
    exact = oracle.prod_f64(o_dia, B, dst, trans, alpha, beta)
    assert_close_mag(got, exact, mag, what + " vs fp64")
    return got, ran


def check_dd2dia(oracle, o_dia, A, B, alpha, beta, path, what):
    got, ran = gpu_dd2dia(o_dia, A, B, alpha, beta, path)
    ref = oracle.dd2dia(o_dia, A, B, alpha, beta)
    valid = oracle.valid_mask(o_dia)
    # padding slots: bit-identical to what dst held before (NaN-aware)
    assert np.array_equal(got[~valid].view(np.uint32), o_dia.vals[~valid].view(np.uint32)), \
        "%s: padding slots were written" % what
    exact = oracle.dd2dia_f64(o_dia, A, B, alpha, beta)
    mag = oracle.dd2dia_f64(
        type(o_dia)(o_dia.h, o_dia.w, o_dia.offsets, o_dia.stride, o_dia.rf, np.abs(o_dia.vals)),
        np.abs(A), np.abs(B), abs(alpha), abs(beta))
    assert_close_mag(got[valid], ref[valid], mag[valid], what)
    assert_close_mag(got[valid], exact[valid], mag[valid], what + " vs fp64")
    return got, ran
