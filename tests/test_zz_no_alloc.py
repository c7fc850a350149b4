"""sbnet_reduce_mask_static, the entry point that allocates nothing (its scratch is an array inside the library's
code object), against sbnet_reduce_mask with a caller's workspace: both through the C ABI, bit-exact, two calls in a
row of which the second is the smaller, so that what the first call left in the shared array is there to be
ignored."""
import ctypes

import numpy as np
import pytest
import torch

from sbnet_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
I2 = ctypes.c_int32 * 2


def both(lib, mask, bcount, bsize, bstride, boffset, tol, avgpool):
    """(indices, count) of sbnet_reduce_mask with a workspace and of sbnet_reduce_mask_static."""
    N, H, W = mask.shape[:3]
    md = torch.from_numpy(mask).to(DEV)
    T = N * bcount[0] * bcount[1]
    bc, bs, bst, bo = I2(*bcount), I2(*bsize), I2(*bstride), I2(*boffset)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        idx = torch.full((T, 3), -7, dtype=torch.int16, device=DEV)
        cnt = torch.full((1,), -1, dtype=torch.int32, device=DEV)
        if static:
            rc = lib.sbnet_reduce_mask_static(md.data_ptr(), N, H, W, bc, 2, bs, 2, bst, 2, bo, 2, tol, int(avgpool),
                                              idx.data_ptr(), cnt.data_ptr(), stream)
        else:
            nws = lib.sbnet_reduce_mask_workspace_bytes(N, bc, 2)
            ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
            rc = lib.sbnet_reduce_mask(md.data_ptr(), N, H, W, bc, 2, bs, 2, bst, 2, bo, 2, tol, int(avgpool),
                                       idx.data_ptr(), None, cnt.data_ptr(), ws.data_ptr(), nws, stream)
        assert rc == _lib.SBNET_OK, lib.sbnet_status_string(rc)
        torch.cuda.synchronize()
        out.append((idx.cpu().numpy(), int(cnt.cpu()[0])))
    return out


@pytest.mark.parametrize("sizes", [
    # (N, H, W), bcount, bsize, bstride, boffset, avgpool -- first the larger problem, then the smaller one
    [((8, 256, 256), (64, 64), (6, 6), (4, 4), (-1, -1), True),      # 32768 blocks: pooling, scan-free compaction
     ((1, 64, 64), (8, 8), (10, 10), (8, 8), (-1, -1), False)],      # 64 blocks: the one-launch mode
    [((1, 800, 800), (32, 32), (27, 27), (25, 25), (-1, -1), False),  # 1024 blocks in one launch
     ((2, 40, 52), (7, 9), (6, 6), (6, 6), (-2, -1), True)],
])
def test_static_scratch_matches_workspace(sizes):
    lib = _lib.load()
    rng = np.random.default_rng(11)
    for (N, H, W), bcount, bsize, bstride, boffset, avgpool in sizes:
        # isolated pixels at a rate that leaves about half of the blocks active
        px = bsize[0] * bsize[1]
        mask = (rng.random((N, H, W, 1)) < 1.0 - 0.5 ** (1.0 / px)).astype(np.float32)
        tol = 0.5 / px if avgpool else 0.5
        (idx_a, cnt_a), (idx_b, cnt_b) = both(lib, mask, bcount, bsize, bstride, boffset, tol, avgpool)
        assert 0 < cnt_a < N * bcount[0] * bcount[1]
        assert cnt_b == cnt_a
        np.testing.assert_array_equal(idx_b, idx_a)   # rows past the count stay untouched (-7) on both sides


def test_static_scratch_rejects_what_it_cannot_hold():
    lib = _lib.load()
    cap = lib.sbnet_reduce_mask_static_max_indices()
    assert 200000 < cap < 2 * 1024 * 1024
    side = int(np.ceil(np.sqrt(cap + 1)))
    bc = I2(side, side)
    assert lib.sbnet_reduce_mask_workspace_bytes(1, bc, 2) > 2 * 1024 * 1024
    one = I2(1, 1)
    fake = ctypes.c_void_p(0x1000)  # never dereferenced: the call fails before any launch
    rc = lib.sbnet_reduce_mask_static(fake, 1, side, side, bc, 2, one, 2, one, 2, I2(0, 0), 2, 0.5, 0, fake, fake, None)
    assert rc == _lib.SBNET_ETOOBIG
    assert b"sbnet_reduce_mask_static_max_indices" in lib.sbnet_status_string(rc)
