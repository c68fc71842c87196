"""The Python surface of the DIA path beyond the products: the host and device
matrix types, element access, conversions, files and the offset-table
generator, as exported by src/cuv_python/export_dia_mat.cpp:113-235.

Host-side behaviour is checked against the reference's fixtures
(dia_mat.cpp:65-119, convert.cpp:110-129) and closed forms; the device parts
(marked gpu) against the host types and the oracle.
"""
import json
import os

import numpy as np
import pytest

from cuv_amd import dia as D
from cuv_amd import io as dia_io

HERE = os.path.dirname(os.path.abspath(__file__))


def _fixtures():
    with open(os.path.join(HERE, "golden", "dia_dense_fixture.json")) as f:
        return json.load(f)


def _seq_host(fx):
    A = D.host_dia_matrix_f(fx["h"], fx["w"], fx["nd"], fx["stride"], fx["rf"])
    A.set_offsets(fx["offsets"])
    A.push(np.arange(fx["nd"] * fx["stride"], dtype=np.float32))
    return A


# ------------------------------------------------------------------ host ---
def test_host_matrix_element_access_matches_fixture():
    for fx in _fixtures():
        A = _seq_host(fx)
        exp = np.asarray(fx["dense"], np.float32)
        assert len(A) == fx["h"] * fx["w"] and A.shape == (fx["h"], fx["w"])
        for i in range(fx["h"]):
            for j in range(fx["w"]):
                on_band = (j - i) in fx["offsets"]
                assert A.has(i, j) == on_band
                assert A(i, j) == exp[i, j]


def test_host_dia_to_dense_matches_fixture():
    for fx in _fixtures():
        A = _seq_host(fx)
        exp = np.asarray(fx["dense"], np.float32)
        assert np.array_equal(D.dia_to_dense(A), exp)
        dst = np.full((fx["h"], fx["w"]), np.nan, np.float32, order="F")
        assert np.array_equal(D.convert(dst, A), exp)
        with pytest.raises(RuntimeError):
            D.convert(np.zeros((fx["h"] + 1, fx["w"]), np.float32), A)


def test_dia_to_dense_steep_diagonals_agrees_with_element_access():
    # row_fact = 4 (the shape of densedense_to_dia.cpp:66-137): every dense
    # entry must be what operator()(i, j) returns, padding never shows
    h, w, rf = 36, 19, 4
    offs = [-3, -2, -1, 0, 1, 2, 3]
    A = D.host_dia_matrix_f(h, w, len(offs), h, rf)
    A.set_offsets(offs)
    A.push(np.arange(len(offs) * h, dtype=np.float32) + 1)
    dense = D.dia_to_dense(A)
    for i in range(h):
        for j in range(w):
            assert dense[i, j] == A(i, j)
            assert (dense[i, j] != 0) == (abs(j - i // rf) <= 3)


def test_set_writes_on_band_only_and_dia_views_storage():
    A = D.host_dia_matrix_f(8, 8, 2, 8)
    A.set_offsets([1, -2])
    A.set(3, 4, 7.5)            # offset 1
    A.set(3, 3, 9.0)            # offset 0: not stored, ignored
    assert A(3, 4) == 7.5 and A(3, 3) == 0.0 and not A.has(3, 3)
    assert A.vec[0 * 8 + 3] == 7.5 and np.count_nonzero(A.vec) == 1
    d = A.dia(-2)
    assert d.size == 8
    d[5] = 2.0                  # a view: element (5, 3)
    assert A(5, 3) == 2.0
    A.set_offset(1, 2)          # second diagonal now has offset 2
    assert A.get_offset(1) == 2 and A.has(0, 2)


def test_dense_layout_rejects_overlapping_columns():
    # an expanded (stride-0) or overlapping as_strided view would make the kernels address batch*rows floats
    # over storage that holds fewer: for dst that is an out-of-bounds write
    import torch
    from cuv_amd import dia as D
    rows = 16
    x = torch.zeros(rows)
    for bad in (x.expand(4, rows), torch.zeros(64).as_strided((4, rows), (8, 1))):
        for name in ("B", "dst"):
            with pytest.raises(ValueError, match="overlapping"):
                D._check_layout(bad, rows, name)
    assert D._check_layout(torch.zeros(4, rows), rows, "B") == (4, rows)
    assert D._check_layout(torch.zeros(4, 24)[:, :rows], rows, "B") == (4, 24)       # a real leading dimension
    assert D._check_layout(x.expand(1, rows), rows, "B") == (1, rows)                # one column: nothing to overlap
    with pytest.raises(ValueError, match="column-major"):
        D._check_layout(torch.zeros(rows, 4).t(), rows, "B")
    with pytest.raises(RuntimeError, match="rows"):
        D._check_layout(torch.zeros(4, rows + 1), rows, "B")


def test_constructor_preconditions():
    with pytest.raises(RuntimeError, match="m_row_fact>0"):
        D.host_dia_matrix_f(4, 4, 1, 4, 0)
    with pytest.raises(RuntimeError, match="m_stride"):
        D.host_dia_matrix_f(8, 6, 1, 5)
    A = D.host_dia_matrix_f(4, 4, 2, 4)
    with pytest.raises(RuntimeError):
        A.set_offsets([0])
    with pytest.raises(RuntimeError):
        A.push(np.zeros(3))


def test_filter_factory_offsets_closed_form():
    # one map: the centred fs x fs window, dy-major (filter_factory.hpp:56-72)
    f = D.filter_factory_float(128, 128, 7, 1, 1)
    exp = [dy * 128 + dx for dy in range(-3, 4) for dx in range(-3, 4)]
    assert f.offsets().tolist() == exp
    A = f.get_dia()
    assert isinstance(A, D.host_dia_matrix_f)
    assert (A.h, A.w, A.num_dia, A.stride) == (16384, 16384, 49, 16384)
    assert A.get_offsets().tolist() == exp and f.dias_per_filter == 49
    # several maps: fs*fs*(out + in - 1) diagonals, blocks px*py apart, the
    # first block (in - 1) maps below the centred one
    g = D.filter_factory_float(6, 5, 3, 2, 3)
    off = g.offsets().reshape(4, 3, 3)
    for m in range(4):
        for i in range(3):
            for j in range(3):
                assert off[m, i, j] == (i - 1) * 6 + (j - 1) + (m - 1) * 30
    B = g.get_dia()
    assert (B.h, B.w, B.num_dia, B.stride) == (60, 90, 36, 90)


def test_extract_filter_collects_a_columns_weights_per_input_map():
    f = D.filter_factory_float(6, 6, 3, 2, 1)
    A = f.get_dia()                         # 72 x 36, 18 diagonals
    col = 14                                # map position (2, 2): a full 3 x 3 window in both input maps
    for i in range(A.h):
        for j in range(A.w):
            A.set(i, j, 1000.0 * i + j)
    got = f.extract_filter(A, col)
    assert got.shape == (9, 2)
    flat = got.reshape(-1)
    for m in range(2):
        rows = [i for i in range(m * 36, (m + 1) * 36) if A.has(i, col)]
        assert len(rows) == 9
        assert flat[m * 9:(m + 1) * 9].tolist() == [1000.0 * i + col for i in rows]


def test_host_matrix_file_round_trip(tmp_path):
    fx = _fixtures()[0]
    A = _seq_host(fx)
    p = str(tmp_path / "a.npz")
    A.save(p)
    B = D.host_dia_matrix_f(1, 1, 1, 1)
    B.load(p)
    assert (B.h, B.w, B.num_dia, B.stride, B.row_fact) == (A.h, A.w, A.num_dia, A.stride, A.row_fact)
    assert np.array_equal(B.get_offsets(), A.get_offsets()) and np.array_equal(B.vec, A.vec)
    assert list(dia_io.load_fields(p).keys()) == list(dia_io.FIELDS)


def test_host_descriptor_is_a_stand_in():
    A = _seq_host(_fixtures()[0])
    assert D.host_block_descriptor_f(A).dia is A


# ---------------------------------------------------------------- device ---
@pytest.mark.gpu
def test_convert_between_host_and_device_and_pull(oracle):
    import torch
    fx = _fixtures()[0]
    H = _seq_host(fx)
    Dv = D.dev_dia_matrix_f(4, 4, 1, 4)             # does not fit: re-created by convert
    D.convert(Dv, H)
    assert (Dv.h, Dv.w, Dv.num_dia, Dv.stride, Dv.row_fact) == (H.h, H.w, H.num_dia, H.stride, H.row_fact)
    assert np.array_equal(Dv.get_offsets(), H.get_offsets())
    assert np.array_equal(Dv.vec.cpu().numpy(), H.vec)
    exp = np.asarray(fx["dense"], np.float32)
    assert np.array_equal(D.pull(Dv), exp)
    # element access on the device type
    assert Dv(3, 4) == exp[3, 4] and Dv(3, 9) == 0.0 and Dv.has(3, 4) and not Dv.has(3, 9)
    Dv.set(3, 4, -1.25)
    Dv.dia(-1)[7] = 5.0                             # element (7, 6)
    H2 = D.host_dia_matrix_f(1, 1, 1, 1)
    D.convert(H2, Dv)
    assert H2(3, 4) == -1.25 and H2(7, 6) == 5.0
    with pytest.raises(TypeError):
        D.convert(H2, H)
    torch.cuda.synchronize()


@pytest.mark.gpu
def test_factory_matrix_on_the_device_multiplies_like_the_oracle(oracle):
    import torch
    from _gpu_util import assert_close_mag
    f = D.filter_factory_float(16, 16, 5, 1, 1)
    A = f.get_dia(device="cuda:0")
    assert isinstance(A, D.dev_dia_matrix_f) and A.num_dia == 25
    rng = np.random.default_rng(5)
    oA = oracle.Dia(A.h, A.w, A.get_offsets().tolist(), A.stride, 1)
    oA.vals[:] = rng.normal(0, 0.1, oA.vals.size).astype(np.float32)
    A.push(oA.vals)
    B = rng.uniform(-1, 1, (A.w, 40)).astype(np.float32)
    dst = torch.empty(40, A.h, device="cuda:0")
    D.prod(dst, A, D.to_device_colmajor(B), "n", "n", 1.0, 0.0)
    Bf = np.asfortranarray(B)
    ref = oracle.prod(oA, Bf, None, "n", 1.0, 0.0)
    mag = oracle.prod_mag(oA, Bf, None, "n", 1.0, 0.0)
    assert_close_mag(D.to_host_colmajor(dst), ref, mag, "factory matrix product")
    # the descriptor follows a changed offset table
    n0 = A.info()["nnz"]
    A.set_offset(0, 1000)                           # moves one diagonal outside the matrix
    assert A.info()["nnz"] < n0


@pytest.mark.gpu
def test_device_matrix_file_round_trip(tmp_path):
    fx = _fixtures()[1]
    A = D.dev_dia_matrix_f(fx["h"], fx["w"], fx["nd"], fx["stride"], fx["rf"])
    A.set_offsets(fx["offsets"])
    A.push(np.arange(fx["nd"] * fx["stride"], dtype=np.float32))
    p = str(tmp_path / "d.npz")
    A.save(p)
    B = D.dev_dia_matrix_f(1, 1, 1, 1)
    B.load(p)
    assert np.array_equal(D.pull(B), np.asarray(fx["dense"], np.float32))
