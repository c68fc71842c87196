"""Loader and ctypes signatures for libcuvdia.so (the C ABI in include/cuvdia.h).

There is no CPU fallback: a missing library, or a call that returns a
negative code, raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcuvdia.so")

OK = 0
EINVAL, ESHAPE, EHIP, ENOMEM, EUNSUPPORTED, ENODEVICE, ETOOLARGE = -1, -2, -3, -4, -5, -6, -7
ACT_NONE, ACT_SIGMOID, ACT_SIGMOID_SAMPLE = 0, 1, 2
PATH_AUTO, PATH_GENERIC, PATH_TILED, PATH_WALK, PATH_TILED_NOWALK, PATH_WINDOW = 0, 1, 2, 3, 4, 5

_lib = None


class CuvDiaError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        msg = "%s: %s" % (what, lib().cuvdia_strerror(code).decode())
        if code == EHIP:
            msg += " (%s)" % lib().cuvdia_last_hip_error().decode()
        super().__init__(msg)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libcuvdia.so is not built (%s); run `make -j6 -C cuv_amd/csrc` "
            "or __graft_entry__.build()" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    c_int, c_ll, c_f, c_vp, c_char = (ctypes.c_int, ctypes.c_longlong, ctypes.c_float,
                                      ctypes.c_void_p, ctypes.c_char)
    ip = ctypes.POINTER(ctypes.c_int)
    L.cuvdia_abi_version.restype = c_int
    L.cuvdia_strerror.restype = ctypes.c_char_p
    L.cuvdia_strerror.argtypes = [c_int]
    L.cuvdia_last_hip_error.restype = ctypes.c_char_p
    L.cuvdia_set_path.argtypes = [c_int]
    L.cuvdia_last_path.restype = c_int
    L.cuvdia_plan_chunks.argtypes = [ip, c_int, c_int, ip, ip, ip, c_int]
    L.cuvdia_plan_chunks_max.argtypes = [ip, c_int, c_int, c_int, ip, ip, ip, c_int]
    L.cuvdia_plan_units.argtypes = [ip, c_int, ip, ip, c_int]
    L.cuvdia_plan_walk.argtypes = [ip, c_int, c_int, c_int, ip, ip, ip, ip]
    L.cuvdia_plan_walk_launch.argtypes = [ip, c_int, c_int, c_int, c_int, c_int, c_int]
    L.cuvdia_plan_walk_launch.restype = c_ll
    L.cuvdia_plan_window_launch.argtypes = [ip, c_int, c_int, c_int, c_int, c_int]
    L.cuvdia_plan_window_launch.restype = c_ll
    L.cuvdia_last_kernel.argtypes = []
    L.cuvdia_last_kernel.restype = ctypes.c_char_p
    L.cuvdia_desc_create.argtypes = [ctypes.POINTER(c_vp), ip, c_int, c_int, c_int, c_int, c_int]
    L.cuvdia_desc_destroy.argtypes = [c_vp]
    L.cuvdia_desc_info.argtypes = [c_vp, ip, ip, ctypes.POINTER(c_ll)]
    L.cuvdia_spmm_f32.argtypes = [c_vp, c_vp, c_vp, c_ll, c_vp, c_ll, c_int, c_char, c_f, c_f, c_vp]
    L.cuvdia_spmm_bias_act_f32.argtypes = [c_vp, c_vp, c_vp, c_ll, c_vp, c_ll, c_int, c_char, c_f, c_f, c_vp, c_int,
                                           c_vp]
    L.cuvdia_spmm_layer_f32.argtypes = [c_vp, c_vp, c_vp, c_ll, c_vp, c_ll, c_int, c_char, c_f, c_f, c_vp, c_int,
                                        ctypes.c_ulonglong, c_vp]
    L.cuvdia_learn_step_weight_decay_f32.argtypes = [c_vp, c_vp, c_ll, c_f, c_f, c_vp]
    L.cuvdia_learn_step_weight_decay_momentum_f32.argtypes = [c_vp, c_vp, c_vp, c_ll, c_f, c_f, c_f, c_vp]
    L.cuvdia_dd2dia_f32.argtypes = [c_vp, c_vp, c_vp, c_ll, c_vp, c_ll, c_int, c_f, c_f, c_vp]
    L.cuvdia_avg_diagonals_f32.argtypes = [c_vp, c_vp, c_vp, c_vp]
    L.cuvdia_spmm_offsets_f32.argtypes = [c_vp, ip, c_int, c_int, c_int, c_int, c_int, c_vp, c_ll,
                                          c_vp, c_ll, c_int, c_char, c_f, c_f, c_vp]
    L.cuvdia_spmm_offsets_noalloc_f32.argtypes = L.cuvdia_spmm_offsets_f32.argtypes
    L.cuvdia_dd2dia_offsets_f32.argtypes = [c_vp, ip, c_int, c_int, c_int, c_int, c_int, c_vp, c_ll,
                                            c_vp, c_ll, c_int, c_f, c_f, c_vp]
    for name in ("cuvdia_set_path", "cuvdia_plan_chunks", "cuvdia_desc_create", "cuvdia_desc_destroy",
                 "cuvdia_desc_info", "cuvdia_spmm_f32", "cuvdia_dd2dia_f32", "cuvdia_spmm_offsets_f32",
                 "cuvdia_dd2dia_offsets_f32", "cuvdia_cache_clear", "cuvdia_spmm_bias_act_f32",
                 "cuvdia_spmm_layer_f32", "cuvdia_learn_step_weight_decay_f32", "cuvdia_avg_diagonals_f32",
                 "cuvdia_plan_units", "cuvdia_plan_walk", "cuvdia_learn_step_weight_decay_momentum_f32", "cuvdia_plan_chunks_max",
                 "cuvdia_spmm_offsets_noalloc_f32"):
        getattr(L, name).restype = c_int
    _lib = L
    return L


def check(code, what):
    if code < 0:
        raise CuvDiaError(code, what)
    return code
