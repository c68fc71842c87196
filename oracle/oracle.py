"""ctypes front end of the CPU oracle (libdia_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg, as the checker -- never by the product.

All dense operands are fp32, column-major, passed as 2-d numpy arrays in
Fortran order (shape (rows, batch)); DIA values are a flat fp32 array of
nd*stride entries, element (i, j) at vals[d*stride + i] with
offsets[d] == j - i//rf (reference: src/cuv/basics/dia_matrix.hpp:228-243).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdia_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int)


def build():
    """Compile the C restatement (gcc, -ffp-contract=off)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "libdia_oracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_dia_get_f32.restype = ctypes.c_float
    return _lib


def _p(a, typ):
    return a.ctypes.data_as(typ) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _colmajor(a):
    a = np.asarray(a, dtype=np.float32)
    if a.ndim == 1:
        a = a.reshape(-1, 1)
    return np.asfortranarray(a)


def _offs(o):
    return np.ascontiguousarray(o, dtype=np.int32)


class Dia:
    """Plain description of a DIA matrix (no behaviour)."""

    def __init__(self, h, w, offsets, stride=None, rf=1, vals=None):
        self.h, self.w, self.rf = int(h), int(w), int(rf)
        self.offsets = _offs(offsets)
        self.nd = int(self.offsets.size)
        self.stride = int(stride if stride is not None else max(h, w))
        if vals is None:
            vals = np.zeros(self.nd * self.stride, np.float32)
        self.vals = _f32(vals).reshape(-1)
        assert self.vals.size == self.nd * self.stride

    def args(self):
        return (self.h, self.w, self.nd, self.stride, self.rf,
                _p(self.offsets, _i32p))


def valid_mask(dia):
    """Boolean mask over vals: True where a matrix element lives (the slots the
    reference's host loops touch), False for padding."""
    m = np.zeros((dia.nd, dia.stride), bool)
    for d, k in enumerate(dia.offsets.tolist()):
        i0 = dia.rf * max(0, -k)
        j0 = max(0, k)
        n = min(dia.h - i0, dia.rf * (dia.w - j0))
        if n > 0:
            m[d, i0:i0 + n] = True
    return m.reshape(-1)


def nnz(dia):
    return int(valid_mask(dia).sum())


def spmv(dia, x, y, trans="n", alpha=1.0, beta=0.0):
    x = _f32(x).reshape(-1)
    y = _f32(y).reshape(-1).copy()
    rc = lib().oracle_spmv_f32(*dia.args(), _p(dia.vals, _f32p), _p(x, _f32p),
                               _p(y, _f32p), ctypes.c_char(trans.encode()),
                               ctypes.c_float(alpha), ctypes.c_float(beta))
    if rc:
        raise RuntimeError("oracle_spmv_f32 rc=%d" % rc)
    return y


def prod(dia, B, dst=None, trans="n", alpha=1.0, beta=0.0):
    """dst = beta*dst + alpha*op(A)*B, fp32, the reference's host order."""
    B = _colmajor(B)
    n_out = dia.w if trans == "t" else dia.h
    n_in = dia.h if trans == "t" else dia.w
    assert B.shape[0] == n_in, (B.shape, n_in)
    batch = B.shape[1]
    if dst is None:
        out = np.full((n_out, batch), np.nan, np.float32, order="F")
        assert beta == 0.0
    else:
        out = _colmajor(dst).copy(order="F")
        assert out.shape == (n_out, batch)
    rc = lib().oracle_prod_dia_f32(*dia.args(), _p(dia.vals, _f32p),
                                   _p(B, _f32p), _p(out, _f32p), batch,
                                   ctypes.c_char(trans.encode()),
                                   ctypes.c_float(alpha), ctypes.c_float(beta))
    if rc:
        raise RuntimeError("oracle_prod_dia_f32 rc=%d" % rc)
    return out


def _prod_shadow(fn, dia, B, dst, trans, alpha, beta):
    B = _colmajor(B)
    n_out = dia.w if trans == "t" else dia.h
    batch = B.shape[1]
    d_in = None if dst is None else _colmajor(dst)
    out = np.zeros((n_out, batch), np.float64, order="F")
    rc = fn(*dia.args(), _p(dia.vals, _f32p), _p(B, _f32p), _p(d_in, _f32p),
            _p(out, _f64p), batch, ctypes.c_char(trans.encode()),
            ctypes.c_float(alpha), ctypes.c_float(beta))
    if rc:
        raise RuntimeError("oracle shadow rc=%d" % rc)
    return out


def prod_f64(dia, B, dst=None, trans="n", alpha=1.0, beta=0.0):
    return _prod_shadow(lib().oracle_prod_dia_f64, dia, B, dst, trans, alpha, beta)


def prod_mag(dia, B, dst=None, trans="n", alpha=1.0, beta=0.0):
    return _prod_shadow(lib().oracle_prod_dia_mag, dia, B, dst, trans, alpha, beta)


def dd2dia_literal(dia, A, B):
    """The reference's host loop as written: C += proj(A*B'), factors ignored."""
    A, B = _colmajor(A), _colmajor(B)
    assert A.shape[0] == dia.h and B.shape[0] == dia.w and A.shape[1] == B.shape[1]
    C = dia.vals.copy()
    rc = lib().oracle_dd2dia_literal_f32(*dia.args(), _p(C, _f32p), _p(A, _f32p),
                                         _p(B, _f32p), A.shape[1])
    if rc:
        raise RuntimeError("oracle_dd2dia_literal_f32 rc=%d" % rc)
    return C


def dd2dia(dia, A, B, alpha=1.0, beta=0.0):
    """Documented contract C = beta*C + alpha*proj(A*B') in the host loop's order."""
    A, B = _colmajor(A), _colmajor(B)
    assert A.shape[0] == dia.h and B.shape[0] == dia.w and A.shape[1] == B.shape[1]
    C = dia.vals.copy()
    rc = lib().oracle_dd2dia_f32(*dia.args(), _p(C, _f32p), _p(A, _f32p),
                                 _p(B, _f32p), A.shape[1],
                                 ctypes.c_float(alpha), ctypes.c_float(beta))
    if rc:
        raise RuntimeError("oracle_dd2dia_f32 rc=%d" % rc)
    return C


def dd2dia_f64(dia, A, B, alpha=1.0, beta=0.0):
    A, B = _colmajor(A), _colmajor(B)
    out = np.zeros(dia.nd * dia.stride, np.float64)
    rc = lib().oracle_dd2dia_f64(*dia.args(), _p(dia.vals, _f32p), _p(out, _f64p),
                                 _p(A, _f32p), _p(B, _f32p), A.shape[1],
                                 ctypes.c_float(alpha), ctypes.c_float(beta))
    if rc:
        raise RuntimeError("oracle_dd2dia_f64 rc=%d" % rc)
    return out


def get(dia, i, j):
    return float(lib().oracle_dia_get_f32(*dia.args(), _p(dia.vals, _f32p), int(i), int(j)))


def to_dense(dia):
    out = np.zeros((dia.h, dia.w), np.float32, order="F")
    lib().oracle_dia_to_dense_f32(*dia.args(), _p(dia.vals, _f32p), _p(out, _f32p))
    return out


def filter_offsets(px, py, fs, input_maps, output_maps):
    n = fs * fs * (output_maps + input_maps - 1)
    out = np.zeros(n, np.int32)
    got = lib().oracle_filter_offsets(px, py, fs, input_maps, output_maps, _p(out, _i32p))
    assert got == n
    return out


def prod_bias_act(dia, B, dst=None, trans="n", alpha=1.0, beta=0.0, bias=None, sigmoid=False):
    """The reference's sequence for a layer update, each step in fp32 as the
    host path does it: prod (spmv.cu:145-220), matrix_plus_col
    (matrix_ops.hpp:307: A(i, j) += v(i)), apply_scalar_functor SIGM
    (functors.hpp:122: 1 / (1 + expf(-t)))."""
    out = prod(dia, B, dst, trans, alpha, beta)
    if bias is not None:
        out = (out + np.asarray(bias, np.float32)[:, None]).astype(np.float32)
    if sigmoid:
        one = np.float32(1)
        out = (one / (one + np.exp(-out, dtype=np.float32))).astype(np.float32)
    return np.asfortranarray(out)


def philox4x32_10(counter, key):
    """Philox4x32-10 of Salmon, Moraes, Dror and Shaw ("Parallel random numbers: as easy as 1, 2, 3", SC'11;
    Random123 1.x, philox.h): counter (..., 4) and key (..., 2) uint32 arrays -> (..., 4) uint32.  The
    algorithm lives in no reference file (the reference samples with cuRAND's XORWOW states,
    src/cuv/random/random.cu:86-91); it is pinned by the known-answer vectors Random123 publishes."""
    c = [np.asarray(counter[..., i], dtype=np.uint64) for i in range(4)]
    k0 = np.asarray(key[..., 0], dtype=np.uint64)
    k1 = np.asarray(key[..., 1], dtype=np.uint64)
    m0, m1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    mask = np.uint64(0xFFFFFFFF)
    sh = np.uint64(32)
    for _ in range(10):
        p0 = m0 * c[0]
        p1 = m1 * c[2]
        c = [(p1 >> sh) ^ c[1] ^ k0, p1 & mask, (p0 >> sh) ^ c[3] ^ k1, p0 & mask]
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return np.stack(c, axis=-1).astype(np.uint32)


def sample_uniform(n_rows, n_cols, seed):
    """u(row, col) in [0, 1): 24 bits of word (col & 3) of the Philox block at counter (row, col >> 2, 0, 0),
    key (seed & 0xffffffff, seed >> 32) -- the draw the fused layer update documents in its header."""
    rows, cols = np.meshgrid(np.arange(n_rows, dtype=np.uint32), np.arange(n_cols, dtype=np.uint32), indexing="ij")
    ctr = np.stack([rows, cols >> 2, np.zeros_like(rows), np.zeros_like(rows)], axis=-1)
    key = np.empty(rows.shape + (2,), np.uint32)
    key[..., 0] = seed & 0xFFFFFFFF
    key[..., 1] = (seed >> 32) & 0xFFFFFFFF
    words = philox4x32_10(ctr, key)
    w = np.take_along_axis(words, (cols & 3)[..., None].astype(np.int64), axis=-1)[..., 0]
    return ((w >> 8).astype(np.float32) * np.float32(2.0 ** -24)).astype(np.float32)


def rnd_binarize(p, u):
    """src/cuv/random/random.cu:86-91: f > uniform, as 0 / 1 floats."""
    return np.asfortranarray((np.asarray(p, np.float32) > np.asarray(u, np.float32)).astype(np.float32))


def learn_step_weight_decay(W, dW, learnrate, decay=0.0):
    """src/cuv/tensor_ops/rprop.cu:331-346: W[i] = alpha*dW[i] + beta*W[i] with alpha = -learnrate and
    beta = 1 - learnrate*decay, every operation rounded to fp32 (sparsedecay is ignored there too)."""
    lr, dc = np.float32(learnrate), np.float32(decay)
    alpha = np.float32(-lr)
    beta = np.float32(np.float32(1) - np.float32(lr * dc))
    W = np.asarray(W, np.float32)
    dW = np.asarray(dW, np.float32)
    return (np.float32(alpha) * dW).astype(np.float32) + (np.float32(beta) * W).astype(np.float32)


def learn_step_weight_decay_momentum(W, momentum, dW, learnrate, momentum_weight=0.9, decay=0.0):
    """src/cuv/tensor_ops/rprop.cu:158-170 (the device kernel; the host loop at rprop.cu:356-367 has the decay
    term's sign flipped): m = momentum_weight*m - learnrate*(dW + decay*W); W += m.  Returns (W, momentum), every
    operation rounded to fp32."""
    f = np.float32
    W, m, dW = (np.asarray(t, f) for t in (W, momentum, dW))
    inner = (dW + (f(decay) * W).astype(f)).astype(f)
    m = ((f(momentum_weight) * m).astype(f) - (f(learnrate) * inner).astype(f)).astype(f)
    return (W + m).astype(f), m


def avg_diagonals(dia):
    out = np.zeros(dia.nd, np.float32)
    lib().oracle_avg_diagonals_f32(dia.h, dia.w, dia.nd, dia.stride,
                                   _p(dia.offsets, _i32p), _p(dia.vals, _f32p),
                                   _p(out, _f32p))
    return out
