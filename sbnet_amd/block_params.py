"""Block-geometry arithmetic: how a convolution's kernel size, stride and padding turn into the
bsize / bstride / boffset / bcount parameters of reduce_mask, sparse_gather and sparse_scatter.

Pure integer arithmetic, no device work.  Follows the reference's
sbnet_tensorflow/benchmark/sparse_conv_lib.py:237-246 (_calc_block_strides), 343-397
(calc_block_params), 400-421 (calc_block_params_res_block) and
sbnet_tensorflow/benchmark/tf_conv_dims.py:94-181, 243-279 (TensorFlow SAME/VALID output size and
padding rules).  Shapes and sizes are 4-element lists in the reference's conventions:
in_size [N,H,W,C], bsize [1,bh,bw,1], ksize [kh,kw,cin,cout], strides [1,sh,sw,1].
"""
import collections

BlockParams = collections.namedtuple("BlockParams", ["bsize", "bsize_out", "boffset", "bcount", "bstrides"])


class BlockParamError(AssertionError, ValueError):
    """The reference reports bad ksize / strides / bsize with assert statements."""


def _ceil_div(a, b):
    return -((-a) // b)


def calc_out_size_1d(in_size, ksize, stride, padding):
    """tf_conv_dims.py:262-279."""
    if padding == "VALID":
        return _ceil_div(in_size - ksize + 1, stride)
    if padding == "SAME":
        return _ceil_div(in_size, stride)
    raise ValueError('Unknown padding method "%s"' % padding)


def calc_out_size_4d(in_shape, ksize, strides, padding):
    """tf_conv_dims.py:243-259."""
    _check(ksize, strides)
    return [in_shape[0], calc_out_size_1d(in_shape[1], ksize[0], strides[1], padding),
            calc_out_size_1d(in_shape[2], ksize[1], strides[2], padding), ksize[3]]


def calc_padding_1d(in_size, out_size, ksize, stride, padding):
    """tf_conv_dims.py:133-156: total padding along one axis."""
    if padding == "VALID":
        return 0
    if padding == "SAME":
        return max((out_size - 1) * stride + ksize - in_size, 0)
    raise ValueError('Unknown padding method "%s"' % padding)


def calc_padding_4d(in_shape, ksize, strides, padding):
    """tf_conv_dims.py:94-130: (pad_top, pad_bottom, pad_left, pad_right); the odd pixel goes last."""
    _check(ksize, strides)
    if padding == "VALID":
        return 0, 0, 0, 0
    if padding != "SAME":
        raise ValueError('Unknown padding method "%s"' % padding)
    out_h = calc_out_size_1d(in_shape[1], ksize[0], strides[1], padding)
    out_w = calc_out_size_1d(in_shape[2], ksize[1], strides[2], padding)
    pad_h = calc_padding_1d(in_shape[1], out_h, ksize[0], strides[1], padding)
    pad_w = calc_padding_1d(in_shape[2], out_w, ksize[1], strides[2], padding)
    return pad_h // 2, pad_h - pad_h // 2, pad_w // 2, pad_w - pad_w // 2


def _check(ksize, strides):
    if len(ksize) != 4:
        raise BlockParamError("Expect `ksize` a list/tuple of length 4.")
    if len(strides) != 4:
        raise BlockParamError("Expect `strides` a list/tuple of length 4.")
    if not (strides[0] == strides[3] == 1):
        raise BlockParamError("Expect first and last dimension of `strides` = 1.")


def calc_block_strides(bsize, ksize, strides):
    """sparse_conv_lib.py:237-246: consecutive blocks overlap by ksize - stride pixels."""
    return [1, bsize[1] - ksize[0] + strides[1], bsize[2] - ksize[1] + strides[2], 1]


def calc_block_params(in_size, bsize, ksize, strides, padding):
    """sparse_conv_lib.py:343-397."""
    if (bsize[1] - ksize[0]) % strides[1] != 0 or (bsize[2] - ksize[1]) % strides[2] != 0:
        raise BlockParamError("Expect `stride` divides `bsize` - `ksize`.")
    bstrides = calc_block_strides(bsize, ksize, strides)
    pad_h0, pad_h1, pad_w0, pad_w1 = calc_padding_4d(in_size, ksize, strides, padding)
    h, w = in_size[1], in_size[2]
    # extend the far-side padding so that blocks tile the padded extent exactly
    pad_h1 += (-h + bsize[1]) % bstrides[1]
    pad_w1 += (-w + bsize[2]) % bstrides[2]
    boffset = [-pad_h0, -pad_w0]
    x_pad_shape = [in_size[0], h + pad_h0 + pad_h1, w + pad_w0 + pad_w1, in_size[3]]
    out_shape = calc_out_size_4d(x_pad_shape, [bsize[1], bsize[2], 1, 1], bstrides, "VALID")
    bcount = [out_shape[1], out_shape[2]]
    bsize_out = calc_out_size_4d(bsize, ksize, strides, "VALID")[1:3]
    for off, st, cnt, siz in zip(boffset, bstrides[1:3], bcount, (h, w)):
        if not off + st * (cnt - 1) < siz:
            raise BlockParamError("last block starts outside the input: boffset %d bstrides %d bcount %d size %d" %
                             (off, st, cnt, siz))
    return BlockParams(bsize=list(bsize[1:3]), bsize_out=list(bsize_out), boffset=boffset, bcount=bcount,
                       bstrides=list(bstrides[1:3]))


def calc_block_params_res_block(in_size, bsize, ksize_list, strides, padding):
    """sparse_conv_lib.py:400-421: a residual block is one convolution with its receptive field as kernel."""
    kh = 1 + sum(k[0] - 1 for k in ksize_list)
    kw = 1 + sum(k[1] - 1 for k in ksize_list)
    return calc_block_params(in_size, bsize, [kh, kw, 1, 1], strides, padding)


def calc_block_count_covering(size, boffset, bstride):
    """Block count along one axis such that the last block still touches one pixel
    (sbnet_tensorflow/sbnet_ops/tests/test_sparse_blocks.py:101-112)."""
    return 1 + (size - boffset - 1) // bstride
