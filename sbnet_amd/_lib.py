"""Loader for libsbnet_amd.so (the C ABI declared in include/sbnet_amd.h).

There is no fallback: if the library has not been built, loading raises.  Build it with
`make -C sbnet_amd/csrc` (or `python -c "import __graft_entry__ as g; g.build()"`).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsbnet_amd.so")

# status codes of include/sbnet_amd.h
SBNET_OK = 0
SBNET_EINVAL_PARAM_SHAPE = 1
SBNET_EINVAL_RANK = 2
SBNET_EINVAL_OVERLAP = 3
SBNET_EINVAL_ARG = 4
SBNET_EHIP = 5
SBNET_ETOOBIG = 6

_vp = ctypes.c_void_p
_int = ctypes.c_int
_i32 = ctypes.c_int32
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_uint = ctypes.c_uint
_sz = ctypes.c_size_t
_f = ctypes.c_float

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "sbnet_status_string": (ctypes.c_char_p, [_int]),
    "sbnet_last_hip_error": (_int, []),
    "sbnet_version": (ctypes.c_char_p, []),
    "sbnet_reduce_mask_max_indices": (ctypes.c_int64, [_int, _i32p, _int]),
    "sbnet_reduce_mask_workspace_bytes": (_sz, [_int, _i32p, _int]),
    "sbnet_reduce_mask": (_int, [_vp, _int, _int, _int, _i32p, _int, _i32p, _int, _i32p, _int, _i32p, _int,
                                 _f, _int, _vp, _i32p, _vp, _vp, _sz, _vp]),
    "sbnet_reduce_mask_static": (_int, [_vp, _int, _int, _int, _i32p, _int, _i32p, _int, _i32p, _int, _i32p, _int,
                                        _f, _int, _vp, _vp, _vp]),
    "sbnet_reduce_mask_static_max_indices": (ctypes.c_int64, []),
    "sbnet_reduce_mask_functor": (_int, [_vp, _int, _int, _int, _f] + [_int] * 8 + [_uint, _uint, _vp, _vp, _int,
                                                                                     _vp, _sz, _vp]),
    "sbnet_sparse_gather": (_int, [_vp, _i64p, _int, _i32, _vp, _i32p, _int, _i32p, _int, _i32p, _int, _int,
                                   _vp, _vp]),
    "sbnet_sparse_gather_functor": (_int, [_vp, _int, _int, _int, _int, _vp] + [_int] * 7 + [_vp, _int, _vp]),
    "sbnet_sparse_gather_grad": (_int, [_vp, _i32, _vp, _vp, _i64p, _int, _i32p, _int, _i32p, _int, _i32p, _int, _int, _vp,
                                        _sz, _vp]),
    "sbnet_sparse_scatter_workspace_bytes": (_sz, [_i32, _i64p, _int, _i32p, _int, _i32p, _int, _i32p, _int]),
    "sbnet_sparse_scatter": (_int, [_vp, _i32, _vp, _vp, _i64p, _int, _i32p, _int, _i32p, _int, _i32p, _int,
                                    _int, _int, _int, _vp, _vp, _sz, _vp]),
    "sbnet_sparse_scatter_var": (_int, [_vp, _i32, _vp, _vp, _i64p, _int, _i32p, _int, _i32p, _int, _i32p, _int,
                                        _int, _int, _int, _vp, _sz, _vp]),
    "sbnet_sparse_scatter_functor": (_int, [_vp, _int, _int, _int, _int, _vp] + [_int] * 7 + [_vp, _int, _int,
                                                                                              _int, _vp]),
    "sbnet_sparse_gather_device_count": (_int, [_vp, _i64p, _int, _vp, _i32, _vp, _i32p, _int, _i32p, _int, _i32p,
                                                _int, _int, _vp, _vp]),
    "sbnet_sparse_scatter_device_count": (_int, [_vp, _vp, _i32, _vp, _vp, _i64p, _int, _i32p, _int, _i32p, _int,
                                                 _i32p, _int, _int, _int, _int, _vp, _vp, _sz, _vp]),
    "sbnet_sparse_scatter_var_device_count": (_int, [_vp, _vp, _i32, _vp, _vp, _i64p, _int, _i32p, _int, _i32p, _int,
                                                     _i32p, _int, _int, _int, _int, _vp, _sz, _vp]),
    "sbnet_sparse_scatter_functor_ws": (_int, [_vp, _int, _int, _int, _int, _vp] + [_int] * 7 + [_vp, _int, _int,
                                                                                                 _int, _vp, _sz, _vp]),
    "sbnet_scratch_acquire": (_vp, [_sz, _vp]),
    "sbnet_shutdown": (_int, []),
    "sbnet_copy_tensor": (_int, [_vp, _vp, _sz, _vp]),
    "sbnet_timer_start": (_int, [_vp, ctypes.POINTER(ctypes.c_int64)]),
    "sbnet_timer_end": (_int, [ctypes.c_int64, _vp, ctypes.POINTER(ctypes.c_float)]),
}

_lib = None


def load():
    """Returns the ctypes handle of libsbnet_amd.so with every entry point typed."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libsbnet_amd.so is not built (%s missing); run `make -C sbnet_amd/csrc`. "
                "There is no CPU or PyTorch fallback for these ops." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
