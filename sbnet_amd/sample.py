"""A single sparse convolution layer on synthetic data, written with the three block ops.

The counterpart of the reference's sbnet_tensorflow/sbnet_ops/sample/sample.py: a [4,256,256,64] input, 16x16
blocks stepping by 14 pixels (so that a 3x3 VALID convolution of a block yields 14x14 outputs that tile the
output), a random block mask at 90 % sparsity.  reduce_mask turns the mask into the list of active blocks,
sparse_gather stacks those blocks channels-first, a dense convolution runs on the stack, and sparse_scatter
writes the results over the VALID-cropped input.  The result is checked against the dense convolution on
the pixels the blocks wrote.

    python -m sbnet_amd.sample
"""
import numpy as np
import torch
import torch.nn.functional as F

import sbnet_amd


def divup(a, b):
    return (a + b - 1) // b


def main(seed=0, device="cuda:0"):
    batch, hw, channels = 4, 256, 64
    block_size, block_stride, block_offset = [16, 16], [14, 14], [0, 0]
    block_count = [divup(hw, block_stride[0]), divup(hw, block_stride[1])]
    in_params = dict(bsize=block_size, boffset=block_offset, bstride=block_stride)
    out_params = dict(bsize=[block_size[0] - 2, block_size[1] - 2], boffset=block_offset, bstride=block_stride)

    rng = np.random.default_rng(seed)
    # attention / a-priori sparsity: one value per block, thresholded at the 90th percentile, upsampled to pixels
    coarse = rng.standard_normal((batch, block_count[0], block_count[1], 1)).astype(np.float32)
    sparse_mask = (coarse > np.percentile(coarse, 90)).astype(np.float32)
    mask = sparse_mask.repeat(block_stride[0], axis=1).repeat(block_stride[1], axis=2)[:, :hw, :hw, :]

    x = torch.from_numpy(rng.standard_normal((batch, hw, hw, channels)).astype(np.float32)).to(device)
    w = torch.from_numpy(rng.standard_normal((3, 3, channels, channels)).astype(np.float32)).to(device)
    mask = torch.from_numpy(np.ascontiguousarray(mask)).to(device)

    # fused pooling + indexing: mask -> list of active blocks
    indices = sbnet_amd.reduce_mask(mask, block_count, tol=0.5, **in_params)
    # active, overlapping tiles stacked along the batch dimension, channels first
    block_stack = sbnet_amd.sparse_gather(x, indices.bin_counts, indices.active_block_indices, transpose=True,
                                          **in_params)
    # dense convolution on the stack of tiles
    conv_blocks = F.conv2d(block_stack, w.permute(3, 2, 0, 1).contiguous())
    # written over the input, which a VALID convolution shrinks by one pixel on each side
    valid_x = x[:, 1:hw - 1, 1:hw - 1, :].contiguous()
    y = sbnet_amd.sparse_scatter(conv_blocks, indices.bin_counts, indices.active_block_indices, valid_x,
                                 transpose=True, add=False, atomic=False, **out_params)

    # check: dense convolution where a block wrote, the input elsewhere
    dense = F.conv2d(x.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1).contiguous()).permute(0, 2, 3, 1)
    wrote = torch.zeros((batch, hw - 2, hw - 2), dtype=torch.bool, device=device)
    n_active = int(indices.bin_counts[0])
    for n, bh, bw in indices.active_block_indices[:n_active].cpu().numpy():
        wrote[n, bh * 14:bh * 14 + 14, bw * 14:bw * 14 + 14] = True
    expect = torch.where(wrote[..., None], dense, valid_x)
    err = float((y - expect).abs().max())
    print("active blocks: %d of %d; output %s; max |sparse - dense| on written pixels: %.3g"
          % (n_active, batch * block_count[0] * block_count[1], tuple(y.shape), err))
    assert err < 1e-2 * float(dense.abs().max())
    return y


if __name__ == "__main__":
    main()
