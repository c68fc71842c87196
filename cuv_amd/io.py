"""Saving and loading DIA matrices.

The reference serialises a host dia_matrix through Boost.Serialization
(src/cuv/basics/sparse_matrix_io.hpp:52-66): the fields m_width, m_height,
m_num_dia, m_stride, m_row_fact, m_offsets and the value vector, in that
order, into a boost::archive::binary_oarchive.  A Boost binary archive is
not a documented interchange format (it carries a library-version header and
is declared non-portable by Boost), no such file ships with the reference and
Boost is not available here, so byte compatibility is not attempted: the same
seven fields, under the same names and in the same order, go into a NumPy
.npz container instead.  `dia_to_fields` / `fields_to_dia` are the device
side: pull to / push from the host, as the reference's Python users do with
`pull` and the constructors (src/cuv_python/export_dia_mat.cpp:113-235).
"""
import numpy as np

FIELDS = ("m_width", "m_height", "m_num_dia", "m_stride", "m_row_fact", "m_offsets", "m_vec")


def check_fields(f):
    """Validates a field dictionary the way the dia_matrix constructor and
    set_offsets do (src/cuv/basics/dia_matrix.hpp:98-109,131,156-175)."""
    missing = [k for k in FIELDS if k not in f]
    if missing:
        raise ValueError("not a DIA matrix file: missing %s" % ", ".join(missing))
    w, h, nd, stride, rf = (int(f[k]) for k in FIELDS[:5])
    if rf <= 0:
        raise RuntimeError("m_row_fact>0")
    if not (stride >= h or stride >= w):
        raise RuntimeError("m_stride >= this->h() || m_stride >= this->w()")
    offs = np.asarray(f["m_offsets"])
    vec = np.asarray(f["m_vec"])
    if offs.ndim != 1 or offs.size != nd or offs.dtype != np.int32:
        raise ValueError("m_offsets must hold m_num_dia int32 entries")
    if vec.ndim != 1 or vec.size != nd * stride or vec.dtype != np.float32:
        raise ValueError("m_vec must hold m_num_dia*m_stride float32 entries")
    return w, h, nd, stride, rf, offs, vec


def save_fields(path, fields):
    """Writes the seven fields, in the reference's order, to `path` (.npz)."""
    check_fields(fields)
    with open(path, "wb") as fh:
        np.savez(fh, **{k: np.asarray(fields[k]) for k in FIELDS})


def load_fields(path):
    with np.load(path, allow_pickle=False) as z:
        f = {k: z[k] for k in z.files}
    check_fields(f)
    return {k: f[k] for k in FIELDS}


def dia_to_fields(A):
    """Device matrix -> host fields (one device-to-host copy of the value vector)."""
    return dict(m_width=np.int64(A.w), m_height=np.int64(A.h), m_num_dia=np.int64(A.num_dia),
                m_stride=np.int64(A.stride), m_row_fact=np.int64(A.row_fact),
                m_offsets=A.get_offsets().astype(np.int32), m_vec=A.pull().astype(np.float32))


def fields_to_dia(fields, device="cuda:0"):
    from .dia import dev_dia_matrix_f
    w, h, nd, stride, rf, offs, vec = check_fields(fields)
    A = dev_dia_matrix_f(h, w, nd, stride, rf, device=device)
    A.set_offsets(offs)
    A.push(vec)
    return A


def save_dia(path, A):
    save_fields(path, dia_to_fields(A))


def load_dia(path, device="cuda:0"):
    return fields_to_dia(load_fields(path), device=device)
