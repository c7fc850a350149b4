"""Sparse convolution layers built on reduce_mask / sparse_gather / sparse_scatter.

Mirrors the user-facing layer functions of the reference's model library,
sbnet_tensorflow/benchmark/sparse_conv_lib.py: `convert_mask_to_indices_custom` (424-459),
`sparse_conv2d_custom` (536-587), `_bottleneck_residual` (677-723), `res_block_bottleneck`
(726-748), `sparse_res_block_bottleneck` (751-824) and `mask_conv2d` (891-911), and its index-list interface
`convert_mask_to_indices` (279-318), `upsample_indices` (249-276), `convert_mask_to_block_indices` (321-340),
`sparse_conv2d` (462-523) and `sparse_conv2d_matmul` (827-888), which the reference computes with TensorFlow's
gather_nd / scatter_nd and which here run on the same block ops.  The three block ops
run the HIP kernels of this package; the dense convolutions, batch norm and ReLU between gather and
scatter are PyTorch's (MIOpen on this hardware), exactly where the reference calls cuDNN.

Conventions follow the reference: activations are NHWC tensors, kernels are [kh, kw, cin, cout],
`strides` and `bsize` are 4-element lists, `data_format='NCHW'` means the block stack is gathered
transposed ([M, C, bh, bw]) so that the convolutions run on planar data without a separate
transpose.  Everything is differentiable through torch.autograd (the block ops through
sbnet_amd.autograd).
"""
import collections

import torch
import torch.nn.functional as F

from . import _lib, block_params, ops

BN_DECAY = 0.999   # tf.contrib.layers.batch_norm defaults used by the reference (sparse_conv_lib.py:600-601)
BN_EPS = 0.001


def convert_mask_to_indices_custom(mask, block_params, tol, avgpool=False):
    """sparse_conv_lib.py:424-459: mask [N,H,W] or [N,H,W,1] -> (active_block_indices, bin_counts)."""
    return ops.reduce_mask(mask, block_params.bcount, block_params.bsize, block_params.bstrides,
                           block_params.boffset, tol=tol, avgpool=avgpool)


def _hwio_to_oihw(w):
    return w.permute(3, 2, 0, 1).contiguous()


def _conv_blocks(p, w, stride, transpose):
    """VALID convolution on a block stack: [M,C,h,w] when transpose else [M,h,w,C]; kernel [kh,kw,cin,cout]."""
    w_ = _hwio_to_oihw(w)
    if transpose:
        return F.conv2d(p, w_, stride=stride)
    q = F.conv2d(p.permute(0, 3, 1, 2), w_, stride=stride)
    return q.permute(0, 2, 3, 1).contiguous()


def sparse_conv2d_custom(x, w, indices, block_params, strides, use_var=False, transpose=False, atomic=False):
    """sparse_conv_lib.py:536-587: gather blocks, VALID-convolve them, write the results over x.

    x [N,H,W,C]; w [kh,kw,C,K] with K == C (the result is pasted into x's shape); returns x with every
    active block's output region replaced by the convolution result.  With use_var the paste happens in
    place on x (which must not require grad), otherwise on a copy."""
    assert strides[1] == strides[2] == 1, "Only accept strides=1"
    p = ops.sparse_gather(x, indices.bin_counts, indices.active_block_indices, block_params.bsize,
                          block_params.bstrides, block_params.boffset, transpose=transpose)
    q = _conv_blocks(p, w, 1, transpose)
    # The reference passes bstrides as the scatter stride in the in-place flavour and bsize_out in the copying
    # one (sparse_conv_lib.py:569-571, 581-583); with the stride-1 convolutions accepted here the two are equal.
    if use_var:
        return ops.sparse_scatter_var(q, indices.bin_counts, indices.active_block_indices, x,
                                      block_params.bsize_out, block_params.bstrides, [0, 0], add=False,
                                      transpose=transpose, atomic=atomic)
    return ops.sparse_scatter(q, indices.bin_counts, indices.active_block_indices, x, block_params.bsize_out,
                              block_params.bsize_out, [0, 0], add=False, transpose=transpose, atomic=atomic)


def mask_conv2d(x, w, mask, strides, padding):
    """sparse_conv_lib.py:891-911: dense convolution with the output masked by the max-pooled mask; the dense
    twin that sparse convolution results are checked against."""
    if mask.dim() == 3:
        mask = mask.unsqueeze(3)
    assert mask.dim() == 4 and mask.shape[3] == 1, "Mask shape must be [N,H,W] or [N,H,W,1]."
    kh, kw = int(w.shape[0]), int(w.shape[1])
    y = _conv_same_or_valid(x.permute(0, 3, 1, 2), _hwio_to_oihw(w), (strides[1], strides[2]), padding)
    m = _pool_same_or_valid(mask.permute(0, 3, 1, 2), (kh, kw), (strides[1], strides[2]), padding)
    return (y * m).permute(0, 2, 3, 1).contiguous()


# ---------------------------------------------------------------------------------------------
# The reference's index-list interface (its TensorFlow-only twin of the custom ops): the same names and
# argument meaning, computed with this package's block ops
# ---------------------------------------------------------------------------------------------

def _pad_amounts(h, w, ksize, strides, padding, bsize=None, bstrides=None):
    """(top, bottom, left, right) zero padding of sparse_conv_lib.py:150-189 (_pad_input): TensorFlow's SAME / VALID
    padding, the far side extended so that the last block fits when block size and strides are given."""
    ph0, ph1, pw0, pw1 = block_params.calc_padding_4d([1, h, w, 1], ksize, strides, padding)
    if bstrides is not None:
        assert bsize is not None, "Must pass in bsize and bstrides together."
        ph1 += (-(h + ph0 + ph1) + bsize[1]) % bstrides[1]
        pw1 += (-(w + pw0 + pw1) + bsize[2]) % bstrides[2]
    return ph0, ph1, pw0, pw1


def upsample_indices(indices, ksize, strides):
    """sparse_conv_lib.py:249-276: block positions [M,3] (n, i, j) of a pooling with window `ksize` and step
    `strides` -> [M, ksize[1], ksize[2], 3], the (n, h, w) of every pixel of each window.  int32."""
    assert indices.dim() == 2, "Expect indices rank = 2"
    assert ksize[0] == ksize[3] == 1, "Expect first and last dimensions of ksize = 1"
    assert strides[0] == strides[3] == 1, "Expect first and last dimensions of strides = 1, {}".format(strides)
    dev = indices.device
    top_left = indices.to(torch.int32) * torch.tensor([1, strides[1], strides[2]], dtype=torch.int32, device=dev)
    r = torch.arange(ksize[1], dtype=torch.int32, device=dev).view(1, -1, 1)
    c = torch.arange(ksize[2], dtype=torch.int32, device=dev).view(1, 1, -1)
    n = top_left[:, 0].view(-1, 1, 1).expand(-1, ksize[1], ksize[2])
    h = top_left[:, 1].view(-1, 1, 1) + r
    w = top_left[:, 2].view(-1, 1, 1) + c
    return torch.stack([n, h.expand(-1, -1, ksize[2]), w.expand(-1, ksize[1], -1)], dim=3)


def convert_mask_to_indices(mask, bsize, ksize, strides, padding, tol):
    """sparse_conv_lib.py:279-318: mask [N,H,W] -> int32 [M,3], the (n, i, j) of the blocks whose maximum over the
    zero-padded mask exceeds tol, in row-major order.  Runs reduce_mask's kernels (max pooling, ordered
    compaction); the list is cut to its length on the host, as tf.where's dynamic shape is."""
    assert mask.dim() == 3, "Expect mask rank = 3"
    assert isinstance(bsize, (list, tuple)), "`bsize` needs to be a list or tuple."
    assert isinstance(ksize, (list, tuple)), "`ksize` needs to be a list or tuple."
    assert isinstance(strides, (list, tuple)), "`strides` needs to be a list or tuple."
    err_div = "Expect `stride` divides `bsize` - `ksize`. stride {}, bsize {}, ksize {}."
    assert (bsize[1] - ksize[0]) % strides[1] == 0, err_div.format(strides[1], bsize[1], ksize[0])
    assert (bsize[2] - ksize[1]) % strides[2] == 0, err_div.format(strides[2], bsize[2], ksize[1])
    assert strides[0] == strides[3] == 1, "Expect first and last dimensions of strides = 1. Dim {}.".format(strides)
    bstrides = block_params.calc_block_strides(bsize, ksize, strides)
    h, w = int(mask.shape[1]), int(mask.shape[2])
    ph0, ph1, pw0, pw1 = _pad_amounts(h, w, ksize, strides, padding, bsize, bstrides)
    bcount = [(h + ph0 + ph1 - bsize[1]) // bstrides[1] + 1, (w + pw0 + pw1 - bsize[2]) // bstrides[2] + 1]
    if mask.shape[0] == 0 or bcount[0] <= 0 or bcount[1] <= 0:
        return torch.zeros((0, 3), dtype=torch.int32, device=mask.device)
    boffset = [-ph0, -pw0]
    if tol < 0:
        # padding zeros exceed a negative tol, pixels outside the image never do: pad for real
        mask = F.pad(mask, (pw0, pw1, ph0, ph1))
        boffset = [0, 0]
    idx, count = ops.reduce_mask_functor(mask.contiguous(), bcount, bsize[1:3], bstrides[1:3], boffset, tol)
    return idx[:int(count.item())].to(torch.int32)


def convert_mask_to_block_indices(mask, bsize, ksize, strides, padding, tol):
    """sparse_conv_lib.py:321-340: mask [N,H,W] -> int32 [M, bsize[1], bsize[2], 3], the pixels (in the padded
    input's coordinates) of every active block."""
    indices = convert_mask_to_indices(mask, bsize, ksize, strides, padding, tol)
    return upsample_indices(indices, bsize, block_params.calc_block_strides(bsize, ksize, strides))


def _rect_origins(blk_indices):
    """int16 (n, h0, w0) rows of the rectangles of a [M,h,w,3] pixel-index tensor, for block ops that step by one
    pixel: block (n, bh, bw) then starts at pixel (boffset + bh, boffset + bw)."""
    assert blk_indices.dim() == 4 and blk_indices.shape[3] == 3, "Expect blk_indices of shape [M, h, w, 3]"
    bh, bw = int(blk_indices.shape[1]), int(blk_indices.shape[2])
    origin = blk_indices[:, 0, 0, :].to(torch.int32)
    if blk_indices.shape[0]:
        want = upsample_indices(origin, [1, bh, bw, 1], [1, 1, 1, 1])
        if not bool((want == blk_indices.to(torch.int32)).all()):
            raise ValueError("blk_indices must list the pixels of axis-aligned rectangles in row-major order")
        lo, hi = int(origin.min()), int(origin.max())
        if lo < 0 or hi > 32767:
            raise ValueError("block positions must lie in [0, 32767]")
    return origin.to(torch.int16).contiguous()


def _scatter_rectangles(q, origins, count, out_shape):
    """tf.scatter_nd of a stack of rectangles into zeros: q [M, qh, qw, K] lands with its top-left pixel at
    origins[m] = (n, h, w); rectangles that meet are summed; pixels outside `out_shape` are dropped."""
    y = torch.zeros(out_shape, dtype=torch.float32, device=q.device)
    if q.shape[0] == 0:
        return y
    geom = ([int(q.shape[1]), int(q.shape[2])], [1, 1], [0, 0])
    if torch.is_grad_enabled() and q.requires_grad:
        return ops.sparse_scatter(q, count, origins, y, *geom, add=True, atomic=True)
    return ops.sparse_scatter_var(q.contiguous(), count, origins, y, *geom, add=True, atomic=True)


def sparse_conv2d(x, w, blk_indices, strides, padding):
    """sparse_conv_lib.py:462-523: convolution evaluated on the rectangles of `blk_indices` only.

    x [N,H,W,C]; w [kh,kw,C,K]; blk_indices int32 [M,h,w,3] as convert_mask_to_block_indices returns them
    (pixels of M rectangles in the zero-padded input's coordinates).  Each rectangle is gathered (pixels of the
    padding read as zeros, so the input is not padded in memory), convolved VALID with `strides`, and its result
    is written at the rectangle's position in a zero tensor of the convolution's output shape [N,H',W',K]."""
    ksize = [int(v) for v in w.shape]
    out_shape = block_params.calc_out_size_4d([int(v) for v in x.shape], ksize, strides, padding)
    origins = _rect_origins(blk_indices)
    M, bh, bw = int(blk_indices.shape[0]), int(blk_indices.shape[1]), int(blk_indices.shape[2])
    if M == 0:
        return torch.zeros(out_shape, dtype=torch.float32, device=x.device)
    ph0, _, pw0, _ = block_params.calc_padding_4d([int(v) for v in x.shape], ksize, strides, padding)
    count = torch.tensor([M], dtype=torch.int32)
    p = ops.sparse_gather(x, count, origins, [bh, bw], [1, 1], [-ph0, -pw0])
    q = _conv_blocks(p, w, (strides[1], strides[2]), False)
    # a rectangle at padded-input pixel (h0, w0) produces the outputs from (h0 // stride, w0 // stride) on
    out_origins = origins.clone()
    out_origins[:, 1] = torch.div(origins[:, 1], strides[1], rounding_mode="floor")
    out_origins[:, 2] = torch.div(origins[:, 2], strides[2], rounding_mode="floor")
    return _scatter_rectangles(q, out_origins, count, out_shape)


def sparse_conv2d_matmul(x, w, blk_indices, strides, padding):
    """sparse_conv_lib.py:827-888: the same for rectangles of exactly the kernel's size and stride 1: every
    rectangle is one output pixel, computed as a matrix product of the gathered patches with the flattened kernel."""
    ksize = [int(v) for v in w.shape]
    if int(blk_indices.shape[1]) != ksize[0] or int(blk_indices.shape[2]) != ksize[1]:
        raise ValueError("Expect blk_indices.shape[1] == w.shape[0] and blk_indices.shape[2] == w.shape[1].")
    if strides[1] != 1 or strides[2] != 1:
        raise ValueError("Strides > 1 not supported.")
    out_shape = block_params.calc_out_size_4d([int(v) for v in x.shape], ksize, strides, padding)
    origins = _rect_origins(blk_indices)
    M = int(blk_indices.shape[0])
    if M == 0:
        return torch.zeros(out_shape, dtype=torch.float32, device=x.device)
    ph0, _, pw0, _ = block_params.calc_padding_4d([int(v) for v in x.shape], ksize, strides, padding)
    count = torch.tensor([M], dtype=torch.int32)
    p = ops.sparse_gather(x, count, origins, [ksize[0], ksize[1]], [1, 1], [-ph0, -pw0])
    q = p.reshape(M, ksize[0] * ksize[1] * ksize[2]) @ w.reshape(ksize[0] * ksize[1] * ksize[2], ksize[3])
    return _scatter_rectangles(q.view(M, 1, 1, ksize[3]), origins, count, out_shape)


def _same_pads(size, k, s):
    out = -(-size // s)
    total = max((out - 1) * s + k - size, 0)
    return total // 2, total - total // 2


def _conv_same_or_valid(x_nchw, w_oihw, stride, padding):
    """TensorFlow's SAME / VALID conventions (the odd padding pixel goes to the bottom/right)."""
    if padding == "SAME":
        ph = _same_pads(x_nchw.shape[2], w_oihw.shape[2], stride[0])
        pw = _same_pads(x_nchw.shape[3], w_oihw.shape[3], stride[1])
        x_nchw = F.pad(x_nchw, (pw[0], pw[1], ph[0], ph[1]))
    elif padding != "VALID":
        raise ValueError('Unknown padding method "%s"' % padding)
    return F.conv2d(x_nchw, w_oihw, stride=stride)


def _pool_same_or_valid(m_nchw, k, stride, padding):
    if padding == "SAME":
        ph = _same_pads(m_nchw.shape[2], k[0], stride[0])
        pw = _same_pads(m_nchw.shape[3], k[1], stride[1])
        m_nchw = F.pad(m_nchw, (pw[0], pw[1], ph[0], ph[1]), value=float("-inf"))
    return F.max_pool2d(m_nchw, k, stride)


# ---------------------------------------------------------------------------------------------
# ResNet bottleneck block, dense and sparse
# ---------------------------------------------------------------------------------------------

BatchNormParams = collections.namedtuple("BatchNormParams", ["gamma", "beta", "moving_mean", "moving_var"])


class BottleneckParams(object):
    """Weights of one bottleneck residual function: three convolutions [kh,kw,cin,cout] (1x1, 3x3, 1x1 in
    the reference's blocks) and the batch norms in front of them.  The reference creates these as TensorFlow
    variables inside _conv / _batch_norm (sparse_conv_lib.py:590-674): truncated-normal kernels with
    stddev sqrt(2 / (kh*kw*cout)), gamma 1, beta 0, moving mean 0, moving variance 1."""

    def __init__(self, ksize_list, device, seed=0, dtype=torch.float32):
        g = torch.Generator(device="cpu").manual_seed(seed)
        self.w = []
        self.bn = []
        for ks in ksize_list:
            std = (2.0 / (ks[0] * ks[1] * ks[3])) ** 0.5
            w = torch.empty(tuple(ks), dtype=dtype)
            torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-2 * std, b=2 * std, generator=g)
            self.w.append(w.to(device).requires_grad_(True))
            cin = ks[2]
            self.bn.append(BatchNormParams(torch.ones(cin, device=device, requires_grad=True),
                                           torch.zeros(cin, device=device, requires_grad=True),
                                           torch.zeros(cin, device=device), torch.ones(cin, device=device)))

    def parameters(self):
        out = list(self.w)
        for b in self.bn:
            out += [b.gamma, b.beta]
        return out


def _batch_norm(x, bn, is_training, channels_first):
    """Fused batch norm with scale (sparse_conv_lib.py:590-602); x is [M,C,h,w] or [M,h,w,C]."""
    xc = x if channels_first else x.permute(0, 3, 1, 2)
    y = F.batch_norm(xc, bn.moving_mean, bn.moving_var, bn.gamma, bn.beta, training=is_training,
                     momentum=1.0 - BN_DECAY, eps=BN_EPS)
    return y if channels_first else y.permute(0, 2, 3, 1)


def _conv_layer(x, w, stride, padding, channels_first):
    xc = x if channels_first else x.permute(0, 3, 1, 2)
    y = _conv_same_or_valid(xc, _hwio_to_oihw(w), (stride, stride), padding)
    return y if channels_first else y.permute(0, 2, 3, 1)


def _bottleneck_residual(x, params, strides, padding, is_training, data_format="NHWC", no_activation=False):
    """sparse_conv_lib.py:677-723: [BN, ReLU,] conv1 (strided) - BN, ReLU, conv2 - BN, ReLU, conv3."""
    cf = data_format == "NCHW"
    s = strides[2]
    if not no_activation:
        x = torch.relu(_batch_norm(x, params.bn[0], is_training, cf))
    x = _conv_layer(x, params.w[0], s, padding, cf)
    x = torch.relu(_batch_norm(x, params.bn[1], is_training, cf))
    x = _conv_layer(x, params.w[1], 1, padding, cf)
    x = torch.relu(_batch_norm(x, params.bn[2], is_training, cf))
    x = _conv_layer(x, params.w[2], 1, padding, cf)
    return x


def res_block_bottleneck(x, params, strides, is_training, data_format="NHWC", w_project=None, no_activation=False):
    """sparse_conv_lib.py:726-748: dense y = x + F(x) with SAME convolutions (x in `data_format`)."""
    x_ = x
    if w_project is not None:
        x_ = _conv_layer(x, w_project, strides[2], "SAME", data_format == "NCHW")
    return x_ + _bottleneck_residual(x, params, strides, "SAME", is_training, data_format, no_activation)


def sparse_res_block_bottleneck(x, params, indices, block_params, strides, is_training, data_format="NHWC",
                                w_project=None, no_activation=False, use_var=False):
    """sparse_conv_lib.py:751-824: y = x + F(x) evaluated on the active blocks only.

    x is NHWC in either data format (as in the reference, `data_format` only selects the layout of the block
    stack: 'NCHW' gathers with transpose=True).  The residual function runs with VALID convolutions on the
    gathered blocks and its output is scatter-added onto x (in place with use_var)."""
    transpose = data_format == "NCHW"
    p = ops.sparse_gather(x, indices.bin_counts, indices.active_block_indices, block_params.bsize,
                          block_params.bstrides, block_params.boffset, transpose=transpose)
    if w_project is not None:
        x = _conv_layer(x, w_project, strides[2], "SAME", False)
    q = _bottleneck_residual(p, params, strides, "VALID", is_training, data_format, no_activation)
    q = q.contiguous()
    fn = ops.sparse_scatter_var if use_var else ops.sparse_scatter
    return fn(q, indices.bin_counts, indices.active_block_indices, x, block_params.bsize_out,
              block_params.bsize_out, [0, 0], add=True, transpose=transpose)


# ---------------------------------------------------------------------------------------------
# Timer twins of the reference's CudaTimerStart / CudaTimerEnd ops
# ---------------------------------------------------------------------------------------------

def hip_timer_start_op():
    """sparse_conv_lib.py:527-529 (CudaTimerStart, sparse_gather.cc:390-428): records an event on the current
    stream and returns the handle to pass to hip_timer_end_op."""
    import ctypes
    lib = _lib.load()
    handle = ctypes.c_int64(0)
    ops._check(lib.sbnet_timer_start(ops._stream(), ctypes.byref(handle)))
    return handle.value


def hip_timer_end_op(start_timer):
    """sparse_conv_lib.py:532-533 (CudaTimerEnd, sparse_gather.cc:430-469): records a second event, waits for
    it and returns the elapsed device time in milliseconds.  The handle is consumed."""
    import ctypes
    lib = _lib.load()
    dt = ctypes.c_float(0.0)
    ops._check(lib.sbnet_timer_end(ctypes.c_int64(start_timer), ops._stream(), ctypes.byref(dt)))
    return dt.value
