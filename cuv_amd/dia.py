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


def _check_layout(t, rows, name):
    """(batch, leading dimension) of a (batch, rows) tensor holding a column-major matrix; raises for layouts
    the kernels cannot address.  Looks at shape and strides only."""
    if t.dim() != 2:
        raise TypeError("%s must be 2-d" % name)
    if t.stride(1) != 1:
        raise ValueError("%s must be column-major: shape (batch, rows) with unit stride along rows" % name)
    if t.shape[1] != rows:
        raise RuntimeError("%s has %d rows, expected %d" % (name, t.shape[1], rows))
    if t.shape[0] > 1:
        # columns closer together than their length overlap (expanded or as_strided views): the kernels
        # would address batch*rows floats over storage that holds fewer
        if t.stride(0) < rows:
            raise ValueError("%s: column stride %d is smaller than its %d rows (overlapping columns)"
                             % (name, t.stride(0), rows))
        return t.shape[0], t.stride(0)
    return t.shape[0], max(rows, 1)


def _check_dense(t, rows, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.dim() == 2):
        raise TypeError("%s must be a 2-d float32 CUDA tensor" % name)
    return _check_layout(t, rows, name)


class _dia_matrix_f:
    """What the host and the device DIA matrix share: shape, offset table with
    its reverse map, element access and files.  Element (i, j) lives at
    vec[d*stride + i] with offsets[d] == j - i//row_fact
    (src/cuv/basics/dia_matrix.hpp:57-276)."""

    def _init_shape(self, h, w, num_dia, stride, row_fact):
        if row_fact <= 0:
            raise RuntimeError("m_row_fact>0")
        if not (stride >= h or stride >= w):
            raise RuntimeError("m_stride >= this->h() || m_stride >= this->w()")
        self.h, self.w, self.num_dia, self.stride, self.row_fact = int(h), int(w), int(num_dia), int(stride), int(row_fact)
        self._offsets = np.zeros(self.num_dia, np.int32)
        self._dia2off = {}

    @property
    def shape(self):
        return (self.h, self.w)

    def __len__(self):
        """Number of matrix entries, h*w (matrix.hpp:103)."""
        return self.h * self.w

    def set_offsets(self, offsets):
        offsets = np.ascontiguousarray(offsets, dtype=np.int32)
        if offsets.size != self.num_dia:
            raise RuntimeError("expected %d offsets" % self.num_dia)
        self._offsets = offsets.copy()
        self.post_update_offsets()

    def post_update_offsets(self):
        """Rebuilds the offset -> table position map; of two equal offsets the
        later position wins (dia_matrix.hpp:181-185)."""
        self._dia2off = {int(o): i for i, o in enumerate(self._offsets)}
        self._offsets_changed()

    def _offsets_changed(self):
        pass

    def set_offset(self, idx, val):
        self._offsets[idx] = val
        self._dia2off[int(val)] = int(idx)
        self._offsets_changed()

    def get_offsets(self):
        return self._offsets.copy()

    def get_offset(self, idx):
        return int(self._offsets[idx])

    def _slot(self, i, j):
        """Position of element (i, j) in the value vector, or None off the band."""
        d = self._dia2off.get(int(j) - int(i) // self.row_fact)
        return None if d is None else d * self.stride + int(i)

    def has(self, i, j):
        """Whether the matrix stores element (i, j) (dia_matrix.hpp:244-251)."""
        return self._slot(i, j) is not None

    def __call__(self, i, j):
        """Element (i, j); 0 off the band (dia_matrix.hpp:236-243)."""
        s = self._slot(i, j)
        return 0.0 if s is None else float(self.vec[s])

    def set(self, i, j, val):
        """Writes element (i, j); silently ignored off the band (dia_matrix.hpp:228-235)."""
        s = self._slot(i, j)
        if s is not None:
            self.vec[s] = val

    def dia(self, k):
        """View of the whole stored diagonal with offset k: `stride` entries,
        padding included (dia_matrix.hpp:205-221)."""
        d = self._dia2off[int(k)]
        return self.vec[d * self.stride:(d + 1) * self.stride]

    def save(self, path):
        """Writes the matrix to a file; a device matrix goes through the host
        (src/cuv_python/export_dia_mat.cpp:90-104)."""
        from . import io
        io.save_fields(path, io.dia_to_fields(self))

    def load(self, path):
        """Replaces shape, offsets and values by the file's."""
        from . import io
        w, h, nd, stride, rf, offs, vec = io.check_fields(io.load_fields(path))
        self._init_shape(h, w, nd, stride, rf)
        self.alloc()
        self.set_offsets(offs)
        self.push(vec)
        return self


class host_dia_matrix_f(_dia_matrix_f):
    """DIA matrix in host memory (a NumPy value vector): the container of the
    reference's host_dia_matrix_f (src/cuv_python/export_dia_mat.cpp:113-150).
    It holds data for conversion, files and element access; products run on the
    device only."""

    def __init__(self, h, w, num_dia, stride, row_fact=1):
        self._init_shape(h, w, num_dia, stride, row_fact)
        self.vec = None
        self.alloc()

    def alloc(self):
        self.vec = np.zeros(self.num_dia * self.stride, np.float32)

    def dealloc(self):
        self.vec = None

    def push(self, host_vals):
        v = np.ascontiguousarray(host_vals, dtype=np.float32).reshape(-1)
        if v.size != self.num_dia * self.stride:
            raise RuntimeError("value vector has %d entries, expected %d" % (v.size, self.num_dia * self.stride))
        self.vec = v.copy()
        return self

    def pull(self):
        return self.vec.copy()


class dev_dia_matrix_f(_dia_matrix_f):
    """DIA matrix in device memory (src/cuv/basics/dia_matrix.hpp:57-276).
    Element access copies one value between device and host, as the
    reference's does (src/cuv/basics/reference.cu:18-28)."""

    def __init__(self, h, w, num_dia, stride, row_fact=1, device="cuda:0"):
        self._desc = None
        self._init_shape(h, w, num_dia, stride, row_fact)
        self._device = device
        self.vec = None
        self.alloc()

    def alloc(self):
        self.vec = torch.zeros(self.num_dia * self.stride, dtype=torch.float32, device=self._device)

    def dealloc(self):
        self._drop_desc()
        self.vec = None

    def __del__(self):
        try:
            self._drop_desc()
        except Exception:
            # interpreter shutdown: torch or the library may already be gone, and the
            # process's device memory goes with it
            pass

    def _drop_desc(self):
        if getattr(self, "_desc", None):
            torch.cuda.synchronize()
            _lib.lib().cuvdia_desc_destroy(self._desc)
            self._desc = None

    def _init_shape(self, h, w, num_dia, stride, row_fact):
        self._drop_desc()
        super()._init_shape(h, w, num_dia, stride, row_fact)

    def _offsets_changed(self):
        self._drop_desc()

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


def _adopt(dst, src):
    """Gives dst the shape of src when they differ, as the reference's
    conversions re-create a destination that does not fit
    (src/cuv/convert/convert.cu:71-112)."""
    if dst.shape != src.shape or dst.row_fact != src.row_fact or dst.vec is None \
            or dst.num_dia != src.num_dia or dst.stride != src.stride:
        dst._init_shape(src.h, src.w, src.num_dia, src.stride, src.row_fact)
        dst.alloc()


def dia_to_dense(src):
    """Host DIA matrix -> dense (h, w) float32 array in column-major (Fortran)
    order: zeros, then every stored diagonal's valid run
    (src/cuv/convert/convert.cu:42-66)."""
    if not isinstance(src, host_dia_matrix_f):
        raise TypeError("dia_to_dense takes a host_dia_matrix_f")
    dense = np.zeros((src.h, src.w), np.float32, order="F")
    rf = src.row_fact
    for o in src._offsets:
        o = int(o)
        i0, j0 = rf * max(0, -o), max(0, o)
        n = min(src.h - i0, rf * (src.w - j0))
        if n <= 0:
            continue
        i = i0 + np.arange(n)
        dense[i, j0 + np.arange(n) // rf] = src.vec[src._dia2off[o] * src.stride + i]
    return dense


def convert(dst, src):
    """The reference's DIA conversions (src/cuv_python/export_dia_mat.cpp:203-208):
    host DIA -> device DIA, device DIA -> host DIA (offset table and value
    vector copied, the destination re-created if it does not fit), and host
    DIA -> dense, where dst is a writable (h, w) float32 NumPy array."""
    if isinstance(dst, _dia_matrix_f) and isinstance(src, _dia_matrix_f):
        if type(dst) is type(src):
            raise TypeError("convert copies between a host and a device DIA matrix")
        _adopt(dst, src)
        dst.set_offsets(src.get_offsets())
        dst.push(src.pull())
        return dst
    if isinstance(dst, np.ndarray) and isinstance(src, host_dia_matrix_f):
        if dst.shape != src.shape or dst.dtype != np.float32:
            raise RuntimeError("dst.shape() == src.shape()")
        dst[...] = dia_to_dense(src)
        return dst
    raise TypeError("unsupported conversion")


def pull(m):
    """Device DIA matrix -> dense host matrix, through a host DIA copy
    (dev_dia_mat2tensor, src/cuv_python/export_dia_mat.cpp:161-170)."""
    if not isinstance(m, dev_dia_matrix_f):
        raise TypeError("pull takes a dev_dia_matrix_f")
    hostdia = host_dia_matrix_f(m.h, m.w, m.num_dia, m.stride, m.row_fact)
    convert(hostdia, m)
    return dia_to_dense(hostdia)


class filter_factory_float:
    """Offset tables of locally connected layers
    (src/cuv/basics/filter_factory.hpp:13-80): an fs x fs window on a px x py
    map, input_maps -> output_maps."""

    def __init__(self, px, py, fs, input_maps, output_maps):
        self.px, self.py, self.fs, self.input_maps, self.output_maps = px, py, fs, input_maps, output_maps
        self.dias_per_filter = 0

    def offsets(self):
        """fs*fs*(output_maps + input_maps - 1) offsets i*px + j + m*px*py, map-major
        then window row then window column, shifted by -(px+1)*(fs//2) -
        (input_maps-1)*px*py (filter_factory.hpp:45-72)."""
        px, py, fs = self.px, self.py, self.fs
        m, i, j = np.meshgrid(np.arange(self.output_maps + self.input_maps - 1), np.arange(fs), np.arange(fs),
                              indexing="ij")
        off = (i * px + j + m * px * py).reshape(-1)
        return (off - (px + 1) * (fs // 2) - (self.input_maps - 1) * px * py).astype(np.int32)

    def get_dia(self, device=None):
        """A zero-valued DIA matrix with that pattern: px*py*input_maps rows,
        px*py*output_maps columns (filter_factory.hpp:43-76).  A host matrix,
        or a device matrix when `device` is given."""
        off = self.offsets()
        n = self.px * self.py
        h, w = n * self.input_maps, n * self.output_maps
        self.dias_per_filter = self.fs * self.fs
        dia = host_dia_matrix_f(h, w, off.size, max(h, w)) if device is None \
            else dev_dia_matrix_f(h, w, off.size, max(h, w), device=device)
        dia.set_offsets(off)
        return dia

    def extract_filter(self, dia, filternumber):
        """The weights that feed column `filternumber`, per input map: a
        (fs*fs, input_maps) row-major array whose flat entry map*fs*fs + k is
        the k-th stored element (ascending row) of that column among the rows
        of input map `map`; filling stops when the array is full.  This is
        what filter_factory.hpp:22-41 sets out to do; its own statement of it
        indexes the result pointer instead of the tensor and cannot be run, so
        no reference output exists for it."""
        if isinstance(dia, dev_dia_matrix_f):
            hostdia = host_dia_matrix_f(dia.h, dia.w, dia.num_dia, dia.stride, dia.row_fact)
            dia = convert(hostdia, dia)
        fs2 = self.fs * self.fs
        mat = np.zeros(fs2 * self.input_maps, np.float32)
        map_size = dia.h // self.input_maps
        for map_num in range(self.input_maps):
            fi = 0
            for i in range(map_size):
                r = i + map_num * map_size
                if not dia.has(r, filternumber):
                    continue
                mat[map_num * fs2 + fi] = dia(r, filternumber)
                fi += 1
                if map_num * fs2 + fi >= mat.size:
                    break
        return mat.reshape(fs2, self.input_maps)


class host_block_descriptor_f:
    """The reference's host descriptor is an empty stand-in
    (src/cuv/matrix_ops/densedense_to_sparse.hpp:53-62); so is this."""

    def __init__(self, dia):
        self.dia = dia


class dev_block_descriptor_f:
    """Kept for signature compatibility with densedense_to_dia(C, bd, A, B, ...)
    (src/cuv/matrix_ops/densedense_to_sparse.hpp:69-105); the run table lives in
    the matrix's own descriptor, so this only pins it."""

    def __init__(self, dia):
        self.dia = dia
        self._desc = dia.desc

    def len(self):
        return self.dia.info()["chunks_n"]

    __len__ = len


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
