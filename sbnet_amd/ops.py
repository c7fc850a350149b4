"""Host-side mirror of the reference's op interface over the C ABI of libsbnet_amd.so.

The reference exposes its ops through `tf.load_op_library` as
`sbnet_module.reduce_mask / sparse_gather / sparse_scatter / sparse_scatter_var`
(sbnet_tensorflow/benchmark/sparse_conv_lib.py:74, 452-459, 547-554, 564-586; op signatures in
sbnet_tensorflow/sbnet_ops/reduce_mask.cc:100-110 and sparse_gather.cc:48-57, 242-268).  The
functions here keep those names, argument names and meanings.  PyTorch supplies device memory and
the current stream only; all computation happens in the HIP kernels behind the C ABI, and there is
no fallback if the library is missing.
"""
import collections
import ctypes

import numpy as np
import torch

from . import _lib

ReduceMaskResult = collections.namedtuple("ReduceMask", ["active_block_indices", "bin_counts"])


class InvalidArgument(ValueError):
    """The reference ops fail with tensorflow's InvalidArgument status; same texts here."""


class HipError(RuntimeError):
    pass


def _check(status):
    if status == _lib.SBNET_OK:
        return
    lib = _lib.load()
    text = lib.sbnet_status_string(status).decode()
    if status == _lib.SBNET_EHIP:
        raise HipError("%s: hipError_t %d" % (text, lib.sbnet_last_hip_error()))
    raise InvalidArgument(text)


def _pair(v):
    """Host int32 parameter vector as (keepalive array, pointer, length); length is checked by the library."""
    if isinstance(v, torch.Tensor):
        v = v.detach().cpu().numpy()
    a = np.ascontiguousarray(np.asarray(v, dtype=np.int32).reshape(-1))
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), int(a.shape[0])


def _dims(t):
    d = list(t.shape) + [1] * max(0, 4 - t.dim())
    a = (ctypes.c_int64 * len(d))(*d)
    return a, t.dim()


def _dev_f32(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.float32:
        raise TypeError("%s must be a float32 tensor on the GPU" % name)
    return t.contiguous()


def _idx_i16(t):
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.int16:
        raise TypeError("active_block_indices must be an int16 tensor on the GPU")
    if t.dim() != 2 or t.shape[1] != 3:
        raise InvalidArgument("active_block_indices must have shape [blocks, 3], got %s" % (tuple(t.shape),))
    return t.contiguous()


def _check_count(M, idx):
    """The kernels read M rows of the list: a count beyond it would read past the allocation (the reference does
    not check this either, sparse_gather.cc:190-192; here it is an error instead of a device fault)."""
    if M < 0 or M > int(idx.shape[0]):
        raise InvalidArgument("bin_counts[0] = %d is outside the block list of %d rows" % (M, int(idx.shape[0])))


def _check_stack(t, M, C, R, S, transpose, name):
    want = (C, R, S) if transpose else (R, S, C)
    if t.dim() != 4 or tuple(int(d) for d in t.shape[1:]) != want or int(t.shape[0]) < M:
        raise InvalidArgument("%s must be a block stack of shape [>=%d, %s], got %s" %
                              (name, M, ", ".join(str(d) for d in want), tuple(t.shape)))


def _count(bin_counts):
    """bin_counts lives in host memory in the reference (reduce_mask.cc:244, sparse_gather.cc:234)."""
    if isinstance(bin_counts, torch.Tensor):
        return int(bin_counts.reshape(-1)[0].item())
    return int(np.asarray(bin_counts).reshape(-1)[0])


def _device_count(bin_counts):
    """A bin_counts that is still on the GPU (reduce_mask(..., sync=False)) selects the entry points that read
    the count on the device; returns the int32 tensor, or None for a host-side count."""
    if isinstance(bin_counts, torch.Tensor) and bin_counts.is_cuda:
        if bin_counts.dtype != torch.int32 or bin_counts.numel() < 1:
            raise TypeError("a device-resident bin_counts must be an int32 tensor with one element")
        return bin_counts
    return None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


_workspaces = {}


def _workspace(device, nbytes):
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def release_workspaces():
    """Drops the scratch buffers the op wrappers keep per (device, stream) between calls (they only ever grow) and
    the library's own (sbnet_shutdown).  Waits for the device; the ops can be used again afterwards."""
    if _workspaces:
        torch.cuda.synchronize()
    _workspaces.clear()
    _check(_lib.load().sbnet_shutdown())


def _param(dynamic, attr, name):
    """The ops take their block parameters as `dynamic_b*` inputs (reduce_mask.cc:100-110, sparse_gather.cc:48-57);
    the reference's README.md:53-107 and sample.py:42-43 spell the same int pairs `bsize=`, `bstride=`, `boffset=`
    (and pass the block count second).  Both spellings are accepted; exactly one must be given."""
    if dynamic is not None and attr is not None:
        raise TypeError("pass either dynamic_%s or %s, not both" % (name, name))
    value = dynamic if dynamic is not None else attr
    if value is None:
        raise TypeError("missing block parameter %s (dynamic_%s)" % (name, name))
    return value


def reduce_mask(mask, dynamic_bcount=None, dynamic_bsize=None, dynamic_bstride=None, dynamic_boffset=None, tol=None,
                avgpool=False, sync=True, bcount=None, bsize=None, bstride=None, boffset=None):
    """ReduceMask (reduce_mask.cc:100-221).

    mask: float32 GPU tensor [N,H,W,1] or [N,H,W].  Returns (active_block_indices, bin_counts):
    int16 GPU tensor [N*bcount[0]*bcount[1], 3] whose first bin_counts[0] rows are the active blocks
    in (n, bh, bw) lexicographic order, and an int32 tensor [1] in host memory.  With sync=False the
    count is left on the device (bin_counts is then a GPU tensor) and the call does not wait.
    """
    lib = _lib.load()
    dynamic_bcount, dynamic_bsize = _param(dynamic_bcount, bcount, "bcount"), _param(dynamic_bsize, bsize, "bsize")
    dynamic_bstride = _param(dynamic_bstride, bstride, "bstride")
    dynamic_boffset = _param(dynamic_boffset, boffset, "boffset")
    if tol is None:
        raise TypeError("reduce_mask: tol is required (the op attribute has no default, reduce_mask.cc:102)")
    mask = _dev_f32(mask, "mask")
    if mask.dim() not in (3, 4) or (mask.dim() == 4 and mask.shape[3] != 1):
        raise InvalidArgument("mask must be [N,H,W,1] (or [N,H,W]), got %s" % (tuple(mask.shape),))
    N, H, W = int(mask.shape[0]), int(mask.shape[1]), int(mask.shape[2])
    bc, bcp, bcl = _pair(dynamic_bcount)
    bs, bsp, bsl = _pair(dynamic_bsize)
    bt, btp, btl = _pair(dynamic_bstride)
    bo, bop, bol = _pair(dynamic_boffset)
    max_idx = lib.sbnet_reduce_mask_max_indices(N, bcp, bcl) if bcl == 2 else 0
    with torch.cuda.device(mask.device):
        idx = torch.empty((max(int(max_idx), 1), 3), dtype=torch.int16, device=mask.device)
        nws = lib.sbnet_reduce_mask_workspace_bytes(N, bcp, bcl) if bcl == 2 else 0
        ws = _workspace(mask.device, nws)
        dev_count = torch.empty(1, dtype=torch.int32, device=mask.device)
        host_count = np.zeros(1, dtype=np.int32)
        hp = host_count.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)) if sync else None
        _check(lib.sbnet_reduce_mask(mask.data_ptr(), N, H, W, bcp, bcl, bsp, bsl, btp, btl, bop, bol,
                                     ctypes.c_float(tol), int(bool(avgpool)), idx.data_ptr(), hp,
                                     dev_count.data_ptr(), ws.data_ptr(), ws.numel(), _stream()))
    if sync:
        return ReduceMaskResult(idx, torch.from_numpy(host_count))
    return ReduceMaskResult(idx, dev_count)


def reduce_mask_functor(mask, bcount, bsize, bstride, boffset, tol, avgpool=False):
    """ReduceMaskFunctor (reduce_mask.h:23-44): the op without its host read-back and without the "no active block"
    fix-up of ReduceMaskOp::Compute (reduce_mask.cc:206-218).  Returns (active_block_indices, count): the int16
    list as reduce_mask returns it and an int32 GPU tensor [1] with the raw count, which can be 0.  Does not wait."""
    lib = _lib.load()
    mask = _dev_f32(mask, "mask")
    if mask.dim() not in (3, 4) or (mask.dim() == 4 and mask.shape[3] != 1):
        raise InvalidArgument("mask must be [N,H,W,1] (or [N,H,W]), got %s" % (tuple(mask.shape),))
    N, H, W = int(mask.shape[0]), int(mask.shape[1]), int(mask.shape[2])
    (bc, bcp, bcl), (bs, _, bsl), (bt, _, btl), (bo, _, bol) = _pair(bcount), _pair(bsize), _pair(bstride), _pair(boffset)
    if not (bcl == bsl == btl == bol == 2):
        _check(_lib.SBNET_EINVAL_PARAM_SHAPE)
    with torch.cuda.device(mask.device):
        max_idx = lib.sbnet_reduce_mask_max_indices(N, bcp, bcl)
        idx = torch.empty((max(int(max_idx), 1), 3), dtype=torch.int16, device=mask.device)
        ws = _workspace(mask.device, lib.sbnet_reduce_mask_workspace_bytes(N, bcp, bcl))
        count = torch.empty(1, dtype=torch.int32, device=mask.device)
        _check(lib.sbnet_reduce_mask_functor(mask.data_ptr(), N, H, W, ctypes.c_float(tol), int(bo[0]), int(bo[1]),
                                             int(bs[0]), int(bs[1]), int(bt[0]), int(bt[1]), int(bc[0]), int(bc[1]),
                                             1, 1, idx.data_ptr(), count.data_ptr(), int(bool(avgpool)),
                                             ws.data_ptr(), ws.numel(), _stream()))
    return idx, count


def sparse_gather(x, bin_counts, active_block_indices, dynamic_bsize=None, dynamic_bstride=None, dynamic_boffset=None,
                  transpose=False, out=None, bsize=None, bstride=None, boffset=None):
    """SparseGather (sparse_gather.cc:48-57, 160-218): x [N,H,W,C] -> [M,bsize[0],bsize[1],C], or
    [M,C,bsize[0],bsize[1]] with transpose=True, M = bin_counts[0]; out-of-image pixels read as 0.
    Differentiable with respect to x (sparse_conv_lib.py:80-107)."""
    dynamic_bsize, dynamic_bstride = _param(dynamic_bsize, bsize, "bsize"), _param(dynamic_bstride, bstride, "bstride")
    dynamic_boffset = _param(dynamic_boffset, boffset, "boffset")
    if torch.is_grad_enabled() and isinstance(x, torch.Tensor) and x.requires_grad:
        if out is not None:
            raise ValueError("out= cannot be combined with a differentiable input")
        from .autograd import SparseGatherFunction
        return SparseGatherFunction.apply(x, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride,
                                          dynamic_boffset, bool(transpose))
    return gather_forward(x, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride, dynamic_boffset,
                          transpose, out)


def gather_forward(x, bin_counts, active_block_indices, dynamic_bsize, dynamic_bstride, dynamic_boffset,
                   transpose=False, out=None):
    """The gather without autograd bookkeeping (what SparseGatherFunction.forward and the gradients call)."""
    lib = _lib.load()
    x = _dev_f32(x, "x")
    idx = _idx_i16(active_block_indices)
    dcount = _device_count(bin_counts)
    # with a device-resident count the stack is sized for the whole list and only its first rows are written
    M = int(idx.shape[0]) if dcount is not None else _count(bin_counts)
    bs, bsp, bsl = _pair(dynamic_bsize)
    bt, btp, btl = _pair(dynamic_bstride)
    bo, bop, bol = _pair(dynamic_boffset)
    dims, rank = _dims(x)
    y = out
    with torch.cuda.device(x.device):
        if rank == 4 and bsl == 2 and btl == 2 and bol == 2:
            # past the checks the library reports in the reference's order: sizes the kernels rely on
            _check_count(M, idx)
            C, R, S = int(x.shape[3]), int(bs[0]), int(bs[1])
            if y is None:
                y = torch.empty((M, C, R, S) if transpose else (M, R, S, C), dtype=torch.float32, device=x.device)
            else:
                if not isinstance(y, torch.Tensor) or y.device != x.device or y.dtype != torch.float32 or \
                        not y.is_contiguous():
                    raise TypeError("out must be a contiguous float32 tensor on the device of x")
                _check_stack(y, M, C, R, S, transpose, "out")
        yp = y.data_ptr() if y is not None else None
        if dcount is not None:
            _check(lib.sbnet_sparse_gather_device_count(x.data_ptr(), dims, rank, dcount.data_ptr(), M, idx.data_ptr(),
                                                        bsp, bsl, btp, btl, bop, bol, int(bool(transpose)), yp,
                                                        _stream()))
        else:
            _check(lib.sbnet_sparse_gather(x.data_ptr(), dims, rank, M, idx.data_ptr(), bsp, bsl, btp, btl, bop, bol,
                                           int(bool(transpose)), yp, _stream()))
    return y


def gather_backward(grad, bin_counts, active_block_indices, x_shape, dynamic_bsize, dynamic_bstride, dynamic_boffset,
                    transpose=False):
    """Gradient of sparse_gather with respect to x (sparse_conv_lib.py:80-107: the reference scatters grad onto
    zeros_like(x) with add=True, atomic=True): a tensor of shape x_shape that is zero where no block lies and holds
    the sum of the blocks of `grad` elsewhere, built without clearing the tensor first."""
    lib = _lib.load()
    grad = _dev_f32(grad, "grad")
    idx = _idx_i16(active_block_indices)
    M = _count(bin_counts)
    bs, bsp, bsl = _pair(dynamic_bsize)
    bt, btp, btl = _pair(dynamic_bstride)
    bo, bop, bol = _pair(dynamic_boffset)
    x_shape = tuple(int(d) for d in x_shape)
    dims = (ctypes.c_int64 * max(len(x_shape), 4))(*(list(x_shape) + [1] * max(0, 4 - len(x_shape))))
    rank = len(x_shape)
    if rank == 4 and bsl == 2 and btl == 2 and bol == 2:
        _check_count(M, idx)
        _check_stack(grad, M, x_shape[3], int(bs[0]), int(bs[1]), transpose, "grad")
    with torch.cuda.device(grad.device):
        dx = torch.empty(x_shape, dtype=torch.float32, device=grad.device)
        ws_ptr, ws_bytes = None, 0
        need = lib.sbnet_sparse_scatter_workspace_bytes(M, dims, rank, bsp, bsl, btp, btl, bop, bol)
        if need:
            ws = _workspace(grad.device, need)
            ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
        _check(lib.sbnet_sparse_gather_grad(grad.data_ptr(), M, idx.data_ptr(), dx.data_ptr(), dims, rank, bsp, bsl, btp,
                                            btl, bop, bol, int(bool(transpose)), ws_ptr, ws_bytes, _stream()))
    return dx


def scatter_forward(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride, dynamic_boffset, add,
                    atomic, transpose, use_var, scratch=True):
    """The scatter without autograd bookkeeping.  scratch=False passes no workspace to the library (hardware
    atomics for overlapping adds, unordered overlapping plain writes, copy-then-scatter): what a caller of the
    C ABI gets who brings none."""
    lib = _lib.load()
    x = _dev_f32(x, "x")
    idx = _idx_i16(active_block_indices)
    dcount = _device_count(bin_counts)
    M = min(int(idx.shape[0]), int(x.shape[0])) if dcount is not None else _count(bin_counts)
    if not isinstance(ybase, torch.Tensor) or not ybase.is_cuda or ybase.dtype != torch.float32:
        raise TypeError("ybase must be a float32 tensor on the GPU")
    if use_var and not ybase.is_contiguous():
        raise TypeError("sparse_scatter_var writes in place and needs a contiguous ybase")
    ybase = ybase.contiguous()
    bs, bsp, bsl = _pair(dynamic_bsize)
    bt, btp, btl = _pair(dynamic_bstride)
    bo, bop, bol = _pair(dynamic_boffset)
    dims, rank = _dims(ybase)
    overlap = bsl == 2 and btl == 2 and (bt[0] < bs[0] or bt[1] < bs[1])
    if rank == 4 and bsl == 2 and btl == 2 and bol == 2 and (atomic or not add or not overlap):
        _check_count(M, idx)
        _check_stack(x, M, int(ybase.shape[3]), int(bs[0]), int(bs[1]), transpose, "x")
    with torch.cuda.device(ybase.device):
        ws_ptr, ws_bytes = None, 0
        if scratch and ((add and atomic) or not use_var or (not add and overlap)):
            # scratch for the atomic-free scatter-add of overlapping blocks, for overlapping plain writes in the
            # CPU functor's order (the block listed last wins), and for building the copying op's output in one
            # pass (uncovered pixels copied, covered ones scattered)
            need = lib.sbnet_sparse_scatter_workspace_bytes(M, dims, rank, bsp, bsl, btp, btl, bop, bol)
            if need:
                ws = _workspace(ybase.device, need)
                ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
        flags = (int(bool(add)), int(bool(atomic)), int(bool(transpose)))
        if use_var:
            if dcount is not None:
                _check(lib.sbnet_sparse_scatter_var_device_count(x.data_ptr(), dcount.data_ptr(), M, idx.data_ptr(),
                                                                 ybase.data_ptr(), dims, rank, bsp, bsl, btp, btl,
                                                                 bop, bol, *flags, ws_ptr, ws_bytes, _stream()))
            else:
                _check(lib.sbnet_sparse_scatter_var(x.data_ptr(), M, idx.data_ptr(), ybase.data_ptr(), dims, rank,
                                                    bsp, bsl, btp, btl, bop, bol, *flags, ws_ptr, ws_bytes,
                                                    _stream()))
            return ybase
        y = torch.empty_like(ybase)
        if dcount is not None:
            _check(lib.sbnet_sparse_scatter_device_count(x.data_ptr(), dcount.data_ptr(), M, idx.data_ptr(),
                                                         ybase.data_ptr(), dims, rank, bsp, bsl, btp, btl, bop, bol,
                                                         *flags, y.data_ptr(), ws_ptr, ws_bytes, _stream()))
        else:
            _check(lib.sbnet_sparse_scatter(x.data_ptr(), M, idx.data_ptr(), ybase.data_ptr(), dims, rank, bsp, bsl,
                                            btp, btl, bop, bol, *flags, y.data_ptr(), ws_ptr, ws_bytes, _stream()))
        return y


def sparse_scatter(x, bin_counts, active_block_indices, ybase, dynamic_bsize=None, dynamic_bstride=None,
                   dynamic_boffset=None, add=None, atomic=False, transpose=False, bsize=None, bstride=None,
                   boffset=None):
    """SparseScatter (sparse_gather.cc:256-268, 286-357): returns copy(ybase) with the blocks of x written
    (add=False), added (add=True) or atomically added (add=True, atomic=True) on top.
    Differentiable with respect to x and ybase (sparse_conv_lib.py:110-147)."""
    dynamic_bsize, dynamic_bstride = _param(dynamic_bsize, bsize, "bsize"), _param(dynamic_bstride, bstride, "bstride")
    dynamic_boffset = _param(dynamic_boffset, boffset, "boffset")
    if add is None:
        raise TypeError("sparse_scatter: add is required (the op attribute has no default, sparse_gather.cc:258)")
    if torch.is_grad_enabled() and ((isinstance(x, torch.Tensor) and x.requires_grad) or
                                    (isinstance(ybase, torch.Tensor) and ybase.requires_grad)):
        from .autograd import SparseScatterFunction
        return SparseScatterFunction.apply(x, bin_counts, active_block_indices, ybase, dynamic_bsize,
                                           dynamic_bstride, dynamic_boffset, bool(add), bool(atomic),
                                           bool(transpose))
    return scatter_forward(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                           dynamic_boffset, add, atomic, transpose, use_var=False)


def sparse_scatter_var(x, bin_counts, active_block_indices, ybase, dynamic_bsize=None, dynamic_bstride=None,
                       dynamic_boffset=None, add=None, atomic=False, transpose=False, bsize=None, bstride=None,
                       boffset=None):
    """SparseScatterVar (sparse_gather.cc:242-254, 335-337): the same, in place on ybase, which is returned.
    The reference registers no gradient for this op (its ybase is a variable reference); neither does this."""
    dynamic_bsize, dynamic_bstride = _param(dynamic_bsize, bsize, "bsize"), _param(dynamic_bstride, bstride, "bstride")
    dynamic_boffset = _param(dynamic_boffset, boffset, "boffset")
    if add is None:
        raise TypeError("sparse_scatter_var: add is required (the op attribute has no default, sparse_gather.cc:244)")
    if torch.is_grad_enabled() and ((isinstance(x, torch.Tensor) and x.requires_grad) or
                                    (isinstance(ybase, torch.Tensor) and ybase.requires_grad)):
        raise NotImplementedError("sparse_scatter_var has no gradient (none is registered for SparseScatterVar "
                                  "in the reference); use sparse_scatter, or call it under torch.no_grad()")
    return scatter_forward(x, bin_counts, active_block_indices, ybase, dynamic_bsize, dynamic_bstride,
                           dynamic_boffset, add, atomic, transpose, use_var=True)
