"""Python surface over the C ABI, mirroring the reference's Boost.Python export
of the DIA path (src/cuv_python/export_dia_mat.cpp:113-235): a device DIA
matrix type, `prod(C, A_dia, B, transA, transB, factAB, factC)` and
`densedense_to_dia(C_dia, bd, A, B, factAB, factC)`.

Dense operands are 2-d torch CUDA tensors holding a column-major matrix, i.e.
a tensor of shape (batch, rows) that is contiguous (`t.t()` is the rows x batch
view).  torch only provides device memory and the stream here.
"""
import ctypes

import numpy as np
import torch

from . import _lib


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check_dense(t, rows, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.dim() == 2):
        raise TypeError("%s must be a 2-d float32 CUDA tensor" % name)
    if t.stride(1) != 1:
        raise ValueError("%s must be column-major: shape (batch, rows) with unit stride along rows" % name)
    if t.shape[1] != rows:
        raise RuntimeError("%s has %d rows, expected %d" % (name, t.shape[1], rows))
    return t.shape[0], max(t.stride(0), rows) if t.shape[0] > 1 else max(rows, 1)


class dev_dia_matrix_f:
    """DIA matrix in device memory: element (i, j) at vec[d*stride + i] with
    offsets[d] == j - i//row_fact (src/cuv/basics/dia_matrix.hpp:57-276)."""

    def __init__(self, h, w, num_dia, stride, row_fact=1, device="cuda:0"):
        if row_fact <= 0:
            raise RuntimeError("m_row_fact>0")
        if not (stride >= h or stride >= w):
            raise RuntimeError("m_stride >= this->h() || m_stride >= this->w()")
        self.h, self.w, self.num_dia, self.stride, self.row_fact = h, w, num_dia, stride, row_fact
        self.vec = torch.zeros(num_dia * stride, dtype=torch.float32, device=device)
        self._offsets = np.zeros(num_dia, np.int32)
        self._desc = None

    def __del__(self):
        self._drop_desc()

    def _drop_desc(self):
        if getattr(self, "_desc", None):
            torch.cuda.synchronize()
            _lib.lib().cuvdia_desc_destroy(self._desc)
            self._desc = None

    def set_offsets(self, offsets):
        offsets = np.ascontiguousarray(offsets, dtype=np.int32)
        if offsets.size != self.num_dia:
            raise RuntimeError("expected %d offsets" % self.num_dia)
        self._offsets = offsets.copy()
        self._drop_desc()

    def get_offsets(self):
        return self._offsets.copy()

    @property
    def desc(self):
        if self._desc is None:
            d = ctypes.c_void_p()
            with torch.cuda.device(self.vec.device):
                _lib.check(_lib.lib().cuvdia_desc_create(
                    ctypes.byref(d), self._offsets.ctypes.data_as(ctypes.POINTER(ctypes.c_int)),
                    self.num_dia, self.h, self.w, self.stride, self.row_fact), "cuvdia_desc_create")
            self._desc = d
        return self._desc

    def info(self):
        cn, ct, nnz = ctypes.c_int(), ctypes.c_int(), ctypes.c_longlong()
        _lib.check(_lib.lib().cuvdia_desc_info(self.desc, ctypes.byref(cn), ctypes.byref(ct),
                                               ctypes.byref(nnz)), "cuvdia_desc_info")
        return dict(chunks_n=cn.value, chunks_t=ct.value, nnz=nnz.value)

    def push(self, host_vals):
        """Host -> device copy of the value vector (convert(dev_dia, host_dia),
        src/cuv/convert/convert.cu:71-90)."""
        v = torch.from_numpy(np.ascontiguousarray(host_vals, dtype=np.float32).reshape(-1))
        if v.numel() != self.vec.numel():
            raise RuntimeError("value vector has %d entries, expected %d" % (v.numel(), self.vec.numel()))
        self.vec.copy_(v)
        return self

    def pull(self):
        return self.vec.cpu().numpy()


class dev_block_descriptor_f:
    """Kept for signature compatibility with densedense_to_dia(C, bd, A, B, ...)
    (src/cuv/matrix_ops/densedense_to_sparse.hpp:69-105); the run table lives in
    the matrix's own descriptor, so this only pins it."""

    def __init__(self, dia):
        self.dia = dia
        self._desc = dia.desc

    def len(self):
        return self.dia.info()["chunks_n"]


def prod(dst, A, B, transA="n", transB="n", factAB=1.0, factC=0.0, sync=True):
    """dst = factC*dst + factAB*op(A)*B (src/cuv/matrix_ops/spmv.cu:221-247)."""
    if transB != "n":
        raise RuntimeError("transB == 'n'")
    if transA not in ("n", "t"):
        raise RuntimeError("transA must be 'n' or 't'")
    n_out, n_in = (A.w, A.h) if transA == "t" else (A.h, A.w)
    bb, ldb = _check_dense(B, n_in, "B")
    bd, ldd = _check_dense(dst, n_out, "dst")
    if bb != bd:
        raise RuntimeError("dst.shape()[1] == B.shape()[1]")
    with torch.cuda.device(dst.device):
        _lib.check(_lib.lib().cuvdia_spmm_f32(
            A.desc, A.vec.data_ptr(), B.data_ptr(), ldb, dst.data_ptr(), ldd, bb,
            transA.encode(), factAB, factC, _stream_ptr()), "cuvdia_spmm_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return dst


def prod_bias_act(dst, A, B, transA="n", factAB=1.0, factC=0.0, bias=None, act=_lib.ACT_NONE, seed=0, sync=True):
    """dst = act(factC*dst + factAB*op(A)*B + bias[row]): prod, matrix_plus_col and the SIGM functor of an
    RBM/MLP layer update in one launch (examples/rbm/base.py:48-54,127-136).  act = ACT_SIGMOID_SAMPLE also
    replaces each probability by a Bernoulli sample of it (rnd_binarize, src/cuv/random/random.cu:139-142),
    drawn from Philox4x32-10 keyed by `seed` and the element's (row, column)."""
    if transA not in ("n", "t"):
        raise RuntimeError("transA must be 'n' or 't'")
    n_out, n_in = (A.w, A.h) if transA == "t" else (A.h, A.w)
    bb, ldb = _check_dense(B, n_in, "B")
    bd, ldd = _check_dense(dst, n_out, "dst")
    if bb != bd:
        raise RuntimeError("dst.shape()[1] == B.shape()[1]")
    if bias is not None and not (isinstance(bias, torch.Tensor) and bias.is_cuda and bias.dtype == torch.float32
                                 and bias.is_contiguous() and bias.numel() == n_out):
        raise RuntimeError("A.shape()[0] == v.size()")
    with torch.cuda.device(dst.device):
        _lib.check(_lib.lib().cuvdia_spmm_layer_f32(
            A.desc, A.vec.data_ptr(), B.data_ptr(), ldb, dst.data_ptr(), ldd, bb, transA.encode(), factAB, factC,
            bias.data_ptr() if bias is not None else None, act, int(seed) & 0xFFFFFFFFFFFFFFFF, _stream_ptr()),
            "cuvdia_spmm_layer_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return dst


def densedense_to_dia(C, bd, A, B, factAB=1.0, factC=0.0, sync=True):
    """C = factC*C + factAB*proj(A*B') on C's stored diagonals
    (src/cuv/matrix_ops/densedense_to_sparse.hpp:107-129)."""
    ba, lda = _check_dense(A, C.h, "A")
    bb, ldb = _check_dense(B, C.w, "B")
    if ba != bb:
        raise RuntimeError("A.shape()[1] == B.shape()[1]")
    with torch.cuda.device(C.vec.device):
        _lib.check(_lib.lib().cuvdia_dd2dia_f32(
            C.desc, C.vec.data_ptr(), A.data_ptr(), lda, B.data_ptr(), ldb, ba,
            factAB, factC, _stream_ptr()), "cuvdia_dd2dia_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return C


def avg_diagonals(dst, A, sync=True):
    """dst[d] = mean of diagonal d of A over its valid slots
    (src/cuv/matrix_ops/diagonals.cu:24-51); dst: float32 CUDA tensor of num_dia entries."""
    if A.row_fact != 1:
        raise RuntimeError("dia.row_fact( )==1")
    if not (isinstance(dst, torch.Tensor) and dst.is_cuda and dst.dtype == torch.float32 and dst.is_contiguous()
            and dst.numel() == A.num_dia):
        raise RuntimeError("dia.num_dia( )==dst.size( )")
    with torch.cuda.device(dst.device):
        _lib.check(_lib.lib().cuvdia_avg_diagonals_f32(A.desc, A.vec.data_ptr(), dst.data_ptr(), _stream_ptr()),
                   "cuvdia_avg_diagonals_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return dst


def learn_step_weight_decay(W, dW, learnrate, decay=0.0, sync=True):
    """W = -learnrate*dW + (1 - learnrate*decay)*W (src/cuv/tensor_ops/rprop.cu:341-346).  W, dW: dev_dia_matrix_f
    (the whole value vector is updated, as the reference's call on dia.vec() does) or float32 CUDA tensors."""
    w = W.vec if isinstance(W, dev_dia_matrix_f) else W
    d = dW.vec if isinstance(dW, dev_dia_matrix_f) else dW
    for t in (w, d):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
            raise RuntimeError("W.ptr() / dW.ptr(): contiguous float32 CUDA tensors")
    if w.numel() != d.numel():
        raise RuntimeError("W.size() == dW.size()")
    with torch.cuda.device(w.device):
        _lib.check(_lib.lib().cuvdia_learn_step_weight_decay_f32(w.data_ptr(), d.data_ptr(), w.numel(),
                                                                 learnrate, decay, _stream_ptr()),
                   "cuvdia_learn_step_weight_decay_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return W


def learn_step_weight_decay_momentum(W, momentum, dW, learnrate, momentum_weight=0.9, decay=0.0, sync=True):
    """m = momentum_weight*momentum - learnrate*(dW + decay*W); W += m; momentum = m
    (src/cuv/tensor_ops/rprop.cu:158-170,369-376).  Operands as in learn_step_weight_decay."""
    w, m, d = (t.vec if isinstance(t, dev_dia_matrix_f) else t for t in (W, momentum, dW))
    for t in (w, m, d):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
            raise RuntimeError("W.ptr() / dW.ptr(): contiguous float32 CUDA tensors")
    if w.numel() != d.numel():
        raise RuntimeError("W.size() == dW.size()")
    if w.numel() != m.numel():
        raise RuntimeError("W.size() == momentum.size()")
    with torch.cuda.device(w.device):
        _lib.check(_lib.lib().cuvdia_learn_step_weight_decay_momentum_f32(
            w.data_ptr(), m.data_ptr(), d.data_ptr(), w.numel(), learnrate, momentum_weight, decay, _stream_ptr()),
            "cuvdia_learn_step_weight_decay_momentum_f32")
        if sync:
            torch.cuda.current_stream().synchronize()
    return W


def to_device_colmajor(a, device="cuda:0"):
    """numpy (rows, batch) array -> torch (batch, rows) contiguous CUDA tensor
    holding the same column-major matrix."""
    a = np.asarray(a, dtype=np.float32)
    if a.ndim == 1:
        a = a.reshape(-1, 1)
    return torch.from_numpy(np.ascontiguousarray(a.T)).to(device)


def to_host_colmajor(t):
    """Inverse of to_device_colmajor: returns a Fortran-ordered (rows, batch) array."""
    return np.asfortranarray(t.detach().cpu().numpy().T)
