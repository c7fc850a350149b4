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
    [((8, 256, 256), (64, 64), (6, 6), (4, 4), (-1, -1), True),      # 32768 blocks: 128 pooling workgroups
     ((1, 64, 64), (8, 8), (10, 10), (8, 8), (-1, -1), False)],      # 64 blocks: one compaction workgroup
    [((1, 800, 800), (32, 32), (27, 27), (25, 25), (-1, -1), False),  # 1024 blocks, a wave per block
     ((2, 40, 52), (7, 9), (6, 6), (6, 6), (-2, -1), True)],
    [((2, 400, 400), (400, 400), (1, 1), (1, 1), (0, 0), False),     # 320 000 one-pixel blocks: more than 1024 pooling
     ((1, 30, 30), (10, 10), (3, 3), (3, 3), (0, 0), True)],         # workgroups, so the counts are scanned first
])
def test_static_scratch_matches_workspace(sizes):
    lib = _lib.load()
    rng = np.random.default_rng(11)
    for (N, H, W), bcount, bsize, bstride, boffset, avgpool in sizes:
        # isolated pixels at a rate that leaves about half of the blocks active
        px = bsize[0] * bsize[1]
        assert lib.sbnet_reduce_mask_workspace_bytes(N, I2(*bcount), 2) <= 2 * 1024 * 1024
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
    # sizes that are no sizes are argument errors, as for sbnet_reduce_mask, not "too big"
    for bad in (I2(-4, 4), I2(4, 0), I2(40000, 1)):
        rc = lib.sbnet_reduce_mask_static(fake, 1, 8, 8, bad, 2, one, 2, one, 2, I2(0, 0), 2, 0.5, 0, fake, fake, None)
        assert rc == _lib.SBNET_EINVAL_ARG
    rc = lib.sbnet_reduce_mask_static(fake, -1, 8, 8, I2(4, 4), 2, one, 2, one, 2, I2(0, 0), 2, 0.5, 0, fake, fake, None)
    assert rc == _lib.SBNET_EINVAL_ARG


def test_static_scratch_pipeline_under_graph_capture():
    """What the entry point is for: reduce_mask with the library's own scratch, then gather and the in-place scatter
    that read the count on the device, captured into one HIP graph (after one call outside capture, which looks the
    scratch array's address up) and replayed on different masks, every replay against the CPU oracle.  The capture
    and the replays allocate no device memory."""
    from oracle import sbnet_oracle as orc
    lib = _lib.load()
    rng = np.random.default_rng(5)
    N, H, W, C = 2, 96, 80, 32
    bcount, bsize, bstride, boffset = (6, 5), (18, 18), (16, 16), (-1, -1)
    bc, bs, bst, bo = I2(*bcount), I2(*bsize), I2(*bstride), I2(*boffset)
    T = N * bcount[0] * bcount[1]
    dims = (ctypes.c_int64 * 4)(N, H, W, C)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    xd = torch.from_numpy(x).to(DEV)
    mask_d = torch.zeros((N, H, W, 1), device=DEV)
    idx = torch.zeros((T, 3), dtype=torch.int16, device=DEV)
    cnt = torch.zeros(1, dtype=torch.int32, device=DEV)
    stack = torch.zeros((T, C, bsize[0], bsize[1]), device=DEV)
    out = torch.zeros((N, H, W, C), device=DEV)

    def enqueue(stream):
        st = ctypes.c_void_p(stream.cuda_stream)
        assert lib.sbnet_reduce_mask_static(mask_d.data_ptr(), N, H, W, bc, 2, bs, 2, bst, 2, bo, 2, 0.5, 0,
                                            idx.data_ptr(), cnt.data_ptr(), st) == 0
        assert lib.sbnet_sparse_gather_device_count(xd.data_ptr(), dims, 4, cnt.data_ptr(), T, idx.data_ptr(), bs, 2,
                                                    bst, 2, bo, 2, 1, stack.data_ptr(), st) == 0
        assert lib.sbnet_sparse_scatter_var_device_count(stack.data_ptr(), cnt.data_ptr(), T, idx.data_ptr(),
                                                         out.data_ptr(), dims, 4, bs, 2, bst, 2, bo, 2, 0, 0, 1, None, 0,
                                                         st) == 0

    enqueue(torch.cuda.current_stream())   # outside capture: first use of the scratch array on this device
    torch.cuda.synchronize()
    # under capture sbnet_reduce_mask refuses what it cannot do there, and leaves the capture valid
    g = torch.cuda.CUDAGraph()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.graph(g):
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.sbnet_reduce_mask(mask_d.data_ptr(), N, H, W, bc, 2, bs, 2, bst, 2, bo, 2, 0.5, 0, idx.data_ptr(), None,
                                   cnt.data_ptr(), None, 0, st)
        assert rc == _lib.SBNET_EHIP    # no workspace: it would have to allocate
        enqueue(torch.cuda.current_stream())
    for rep in range(3):
        mask = (rng.random((N, H, W, 1)) < 0.002 * (rep + 1)).astype(np.float32)
        mask_d.copy_(torch.from_numpy(mask))
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        idx_o, cnt_o = orc.reduce_mask(mask, bcount, bsize, bstride, boffset, 0.5, False)
        M = int(cnt_o[0])
        assert int(cnt.cpu()[0]) == M and 0 < M < T
        np.testing.assert_array_equal(idx.cpu().numpy()[:M], idx_o[:M])
        g_o = orc.sparse_gather(x, cnt_o, idx_o, bsize, bstride, boffset, transpose=True)
        np.testing.assert_array_equal(stack.cpu().numpy()[:M], g_o)
        y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, np.zeros_like(x), bsize, bstride, boffset, add=False, transpose=True)
        np.testing.assert_array_equal(out.cpu().numpy(), y_o)
    assert torch.cuda.mem_get_info()[0] >= free_before - (4 << 20)   # (the graph object itself; no buffers)
