"""ctypes front end of the CPU oracle (oracle/sbnet_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg, never by the sbnet_amd package.  Arrays in and out are numpy, C-contiguous.

The functions keep the reference's op names and argument meaning
(sbnet_tensorflow/sbnet_ops/reduce_mask.cc:100-110, sparse_gather.cc:48-57, 242-268).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libsbnet_oracle.so")


class InvalidArgument(ValueError):
    """Mirror of the InvalidArgument status the reference ops raise."""


def build(force=False):
    """Compile the C restatement with gcc (seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "sbnet_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i16p = ctypes.POINTER(ctypes.c_int16)
_i32p = ctypes.POINTER(ctypes.c_int32)
_int = ctypes.c_int


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.oracle_reduce_mask.restype = _int
        L.oracle_reduce_mask.argtypes = [_f32p, _int, _int, _int, ctypes.c_float, _i32p, _i32p, _i32p,
                                         _i32p, _int, _i16p, _i32p]
        g = [_f32p, _int, _int, _int, _int, _f32p] + [_int] * 7 + [_i16p, _int]
        for name in ("oracle_sparse_gather", "oracle_sparse_gather_omp"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = g
        s = [_f32p, _int, _int, _int, _int, _f32p] + [_int] * 7 + [_i16p, _int, _int, _int]
        for name in ("oracle_sparse_scatter", "oracle_sparse_scatter_omp"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = s
        L.oracle_sparse_scatter_op.restype = _int
        L.oracle_sparse_scatter_op.argtypes = [_f32p, _int, _i16p, _f32p, _int, _int, _int, _int, _int,
                                               _i32p, _i32p, _i32p, _int, _int, _int, _int, _f32p]
        _lib = L
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _pair(v, name):
    a = np.asarray(v, dtype=np.int32)
    if a.ndim != 1 or a.shape[0] != 2:
        raise InvalidArgument("dynamic_b<count, size, stride, offset> should be one-dimensional "
                              "with shape[0] == 2. (%s)" % name)
    a = np.ascontiguousarray(a)
    return a, a.ctypes.data_as(_i32p)


def reduce_mask(mask, dynamic_bcount, dynamic_bsize, dynamic_bstride, dynamic_boffset, tol,
                avgpool=False):
    """reduce_mask.cc:123-221.  mask [N,H,W,1] (or [N,H,W]).  Returns (active_block_indices
    int16 [N*bCntH*bCntW, 3], bin_counts int32 [1]); rows past bin_counts[0] are zero here,
    unspecified in the reference."""
    bc, bcp = _pair(dynamic_bcount, "bcount")
    bs, bsp = _pair(dynamic_bsize, "bsize")
    bst, bstp = _pair(dynamic_bstride, "bstride")
    bo, bop = _pair(dynamic_boffset, "boffset")
    m, mp = _f32(mask)
    N, H, W = m.shape[0], m.shape[1], m.shape[2]
    max_idx = N * int(bc[0]) * int(bc[1])
    idx = np.zeros((max(max_idx, 1), 3), dtype=np.int16)
    cnt = np.zeros(1, dtype=np.int32)
    lib().oracle_reduce_mask(mp, N, H, W, ctypes.c_float(tol), bcp, bsp, bstp, bop, int(bool(avgpool)),
                             idx.ctypes.data_as(_i16p), cnt.ctypes.data_as(_i32p))
    return idx[:max(max_idx, 1)], cnt


def sparse_gather(x, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride,
                  dynamic_boffset, transpose=False, omp=False):
    """sparse_gather.cc:160-218.  x [N,H,W,C] -> [M,R,S,C] or [M,C,R,S]."""
    x = np.asarray(x)
    if x.ndim != 4:
        raise InvalidArgument("x must be rank 4")
    bs, _ = _pair(dynamic_bsize, "bsize")
    bst, _ = _pair(dynamic_bstride, "bstride")
    bo, _ = _pair(dynamic_boffset, "boffset")
    xa, xp = _f32(x)
    N, H, W, C = xa.shape
    M = int(np.asarray(bin_counts).reshape(-1)[0])
    R, S = int(bs[0]), int(bs[1])
    y = np.empty((M, C, R, S) if transpose else (M, R, S, C), dtype=np.float32)
    idx = np.ascontiguousarray(active_block_indices, dtype=np.int16)
    fn = lib().oracle_sparse_gather_omp if omp else lib().oracle_sparse_gather
    fn(xp, N, H, W, C, y.ctypes.data_as(_f32p), int(bo[0]), int(bo[1]), R, S, int(bst[0]), int(bst[1]),
       M, idx.ctypes.data_as(_i16p), int(bool(transpose)))
    return y


def _scatter(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
             dynamic_boffset, add, atomic, transpose, use_var):
    bs, bsp = _pair(dynamic_bsize, "bsize")
    bst, bstp = _pair(dynamic_bstride, "bstride")
    bo, bop = _pair(dynamic_boffset, "boffset")
    xa, xp = _f32(x)
    M = int(np.asarray(bin_counts).reshape(-1)[0])
    idx = np.ascontiguousarray(active_block_indices, dtype=np.int16)
    if use_var:
        if not (isinstance(ybase, np.ndarray) and ybase.dtype == np.float32 and ybase.flags.c_contiguous):
            raise TypeError("sparse_scatter_var needs a C-contiguous float32 ndarray to mutate")
        yb = ybase
    else:
        yb = np.ascontiguousarray(ybase, dtype=np.float32)
    dims = list(yb.shape[:4]) + [1] * (4 - min(yb.ndim, 4))
    y = yb if use_var else np.empty_like(yb)
    rc = lib().oracle_sparse_scatter_op(xp, M, idx.ctypes.data_as(_i16p), yb.ctypes.data_as(_f32p),
                                        yb.ndim, dims[0], dims[1], dims[2], dims[3], bsp, bstp, bop,
                                        int(bool(add)), int(bool(atomic)), int(bool(transpose)),
                                        int(bool(use_var)), y.ctypes.data_as(_f32p))
    if rc == 2:
        raise InvalidArgument("ybase must be rank 4")
    if rc != 0:
        raise InvalidArgument("Only non-overlapping blocks are supported with add=True, atomic=False")
    return y


def sparse_scatter(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                   dynamic_boffset, add, atomic=False, transpose=False):
    """sparse_gather.cc:286-357 with UseVar=false: returns a new array = copy(ybase) + scatter."""
    return _scatter(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                    dynamic_boffset, add, atomic, transpose, use_var=False)


def sparse_scatter_var(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                       dynamic_boffset, add, atomic=False, transpose=False):
    """sparse_gather.cc:286-357 with UseVar=true: mutates ybase in place and returns it."""
    return _scatter(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                    dynamic_boffset, add, atomic, transpose, use_var=True)


def sparse_scatter_raw(x, M, idx, y, bsize, bstride, boffset, add, transpose, omp=False):
    """Functor-level scatter into y in place (for timing: no validation, no copy)."""
    fn = lib().oracle_sparse_scatter_omp if omp else lib().oracle_sparse_scatter
    x = np.ascontiguousarray(x, dtype=np.float32)
    idx = np.ascontiguousarray(idx, dtype=np.int16)
    assert y.dtype == np.float32 and y.flags.c_contiguous
    N, H, W, C = y.shape
    fn(x.ctypes.data_as(_f32p), N, H, W, C, y.ctypes.data_as(_f32p), int(boffset[0]), int(boffset[1]),
       int(bsize[0]), int(bsize[1]), int(bstride[0]), int(bstride[1]), int(M),
       idx.ctypes.data_as(_i16p), int(bool(add)), int(bool(transpose)), 0)
    return y


# ---------------------------------------------------------------------------------------------
# Gradients of the two differentiable ops, as the reference registers them
# (sbnet_tensorflow/benchmark/sparse_conv_lib.py:80-147, sbnet_ops/tests/test_sparse_blocks.py:36-98):
# compositions of the forward ops above, nothing else.
# ---------------------------------------------------------------------------------------------

def sparse_gather_grad(grad, x_shape, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride,
                       dynamic_boffset, transpose=False):
    """d(SparseGather)/dx (sparse_conv_lib.py:80-107): the block-shaped gradient scattered with
    add=True, atomic=True onto zeros of x's shape, same transpose as the forward op."""
    zeros = np.zeros(x_shape, dtype=np.float32)
    return sparse_scatter(grad, bin_counts, active_block_indices, zeros, dynamic_bsize, dynamic_bstride,
                          dynamic_boffset, add=True, atomic=True, transpose=transpose)


def sparse_scatter_grad(grad, blocks_shape, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride,
                        dynamic_boffset, add, transpose=False):
    """(d/dblocks, d/dybase) of SparseScatter (sparse_conv_lib.py:110-147).

    d/dblocks = sparse_gather(grad).  The reference calls the gather without the op's transpose attribute,
    which yields an [M,R,S,C]-shaped gradient for an [M,C,R,S] input; here the gather takes the forward op's
    transpose so the gradient has the input's layout (identical to the reference for transpose=False).
    d/dybase = grad for add=True; for add=False grad times the stamp-out mask obtained by scattering blocks
    of zeros over ones."""
    d_blocks = sparse_gather(grad, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride,
                             dynamic_boffset, transpose=transpose)
    if add:
        return d_blocks, grad.copy()
    stamp = sparse_scatter(np.zeros(blocks_shape, dtype=np.float32), bin_counts, active_block_indices,
                           np.ones_like(grad), dynamic_bsize, dynamic_bstride, dynamic_boffset, add=False,
                           transpose=transpose)
    return d_blocks, grad * stamp
