"""Gradients of SparseGather and SparseScatter as torch.autograd.Functions over the C ABI.

The reference registers them in Python as compositions of its own ops
(sbnet_tensorflow/benchmark/sparse_conv_lib.py:80-147, the same text in
sbnet_ops/tests/test_sparse_blocks.py:36-98); the same compositions are used here, so every
backward pass runs the HIP kernels of the forward ops:

* d SparseGather / dx       = sparse_scatter(grad, ..., zeros_like(x), add=True, atomic=True, transpose),
                              computed by one entry point that writes zeros only where no block lies
* d SparseScatter / dblocks = sparse_gather(grad, ...)
* d SparseScatter / dybase  = grad                       (add=True)
                            = grad * stamp-out mask      (add=False; mask = blocks of zeros scattered over ones)

No gradient flows to the index list, the count or the block parameters, as in the reference.

One deliberate difference: the reference calls the gather of d/dblocks without the op's transpose
attribute (sparse_conv_lib.py:124-130), which returns an [M,R,S,C]-shaped gradient for an
[M,C,R,S]-shaped input.  Here the gather uses the forward op's transpose so that the gradient has
the layout of the input; for transpose=False the two coincide.
"""
import torch

from . import ops


def _count_host(bin_counts):
    """The count is read once in forward and kept as a host integer for backward."""
    return ops._count(bin_counts)


class SparseGatherFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bin_counts, active_block_indices, bsize, bstride, boffset, transpose):
        M = _count_host(bin_counts)
        ctx.params = (M, tuple(int(v) for v in ops._pair(bsize)[0]), tuple(int(v) for v in ops._pair(bstride)[0]),
                      tuple(int(v) for v in ops._pair(boffset)[0]), transpose)
        ctx.x_shape = tuple(x.shape)
        ctx.save_for_backward(active_block_indices)
        return ops.gather_forward(x.detach(), [M], active_block_indices, bsize, bstride, boffset, transpose)

    @staticmethod
    def backward(ctx, grad):
        M, bsize, bstride, boffset, transpose = ctx.params
        (idx,) = ctx.saved_tensors
        # the reference scatters onto zeros_like(x) with the copying op; the library builds the same tensor without
        # materialising the zeros first (sbnet_sparse_gather_grad)
        dx = ops.gather_backward(grad.contiguous(), [M], idx, ctx.x_shape, bsize, bstride, boffset, transpose)
        return dx, None, None, None, None, None, None


class SparseScatterFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bin_counts, active_block_indices, ybase, bsize, bstride, boffset, add, atomic, transpose):
        M = _count_host(bin_counts)
        ctx.params = (M, tuple(int(v) for v in ops._pair(bsize)[0]), tuple(int(v) for v in ops._pair(bstride)[0]),
                      tuple(int(v) for v in ops._pair(boffset)[0]), add, transpose)
        ctx.blocks_shape = tuple(x.shape)
        ctx.save_for_backward(active_block_indices)
        return ops.scatter_forward(x.detach(), [M], active_block_indices, ybase.detach(), bsize, bstride, boffset,
                                   add, atomic, transpose, use_var=False)

    @staticmethod
    def backward(ctx, grad):
        M, bsize, bstride, boffset, add, transpose = ctx.params
        (idx,) = ctx.saved_tensors
        grad = grad.contiguous()
        d_blocks = d_ybase = None
        if ctx.needs_input_grad[0]:
            d_blocks = ops.gather_forward(grad, [M], idx, bsize, bstride, boffset, transpose)
        if ctx.needs_input_grad[3]:
            if add:
                d_ybase = grad
            else:
                stamp = torch.ones_like(grad)
                zeros = torch.zeros(ctx.blocks_shape, dtype=torch.float32, device=grad.device)
                ops.scatter_forward(zeros, [M], idx, stamp, bsize, bstride, boffset, add=False, atomic=False,
                                    transpose=transpose, use_var=True)
                d_ybase = grad * stamp
        return d_blocks, None, None, d_ybase, None, None, None, None, None, None
