"""Gradients of SparseGather / SparseScatter (the first "next" component after the three ops).

The reference defines them as compositions of its own ops (benchmark/sparse_conv_lib.py:80-147) and checks
them numerically with TensorFlow's gradient_checker (sbnet_ops/tests/test_sparse_blocks.py:264-284).  Both ops
are linear in their differentiable inputs, so the check here is exact instead of numeric: the Jacobian of the
oracle's FORWARD op is built column by column from basis vectors and its transpose applied to a random
cotangent must equal what the gradient composition returns.  Nothing in that comparison re-types the
composition.  The GPU tests then compare sbnet_amd's autograd Functions with the oracle's gradients.
"""
import numpy as np
import pytest
import torch

from oracle import sbnet_oracle as orc

CASES = [
    # (N, H, W, C), bsize, bstride, boffset
    ((1, 7, 8, 2), (3, 3), (3, 3), (0, 0)),       # tiling, no overlap
    ((2, 7, 8, 1), (3, 4), (2, 3), (-1, -2)),     # overlapping, off-image borders
    ((1, 6, 6, 3), (2, 2), (3, 3), (1, 0)),       # gaps between blocks
    ((1, 5, 9, 2), (4, 4), (2, 2), (-1, -1)),     # up to 2x2 blocks per pixel
]


def setup_case(case, seed, frac=0.7):
    (N, H, W, C), bs, bst, bo = case
    rng = np.random.default_rng(seed)
    bc = [1 + (H - bo[0] - 1) // bst[0], 1 + (W - bo[1] - 1) // bst[1]]
    cells = rng.random((N, bc[0], bc[1])) < frac
    cells[0, 0, 0] = True
    idx = np.ascontiguousarray(np.argwhere(cells), dtype=np.int16)
    cnt = np.array([idx.shape[0]], dtype=np.int32)
    return rng, idx, cnt


def jacobian(fn, n_in):
    """Dense Jacobian of a linear map given as a function of a flat float32 vector."""
    cols = []
    base = fn(np.zeros(n_in, dtype=np.float32)).astype(np.float64).ravel()
    for i in range(n_in):
        e = np.zeros(n_in, dtype=np.float32)
        e[i] = 1.0
        cols.append(fn(e).astype(np.float64).ravel() - base)
    return np.stack(cols, axis=1)  # [n_out, n_in]


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d" % (c[1] + c[2]))
def test_oracle_gather_grad_is_jacobian_transpose(case, transpose):
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 3)
    n_in = int(np.prod(shape))
    J = jacobian(lambda v: orc.sparse_gather(v.reshape(shape), cnt, idx, bs, bst, bo, transpose=transpose), n_in)
    out_shape = orc.sparse_gather(np.zeros(shape, np.float32), cnt, idx, bs, bst, bo, transpose=transpose).shape
    # small integers: every sum below is exact in fp32, so the comparison needs no tolerance
    g = rng.integers(-8, 9, size=out_shape).astype(np.float32)
    dx = orc.sparse_gather_grad(g, shape, cnt, idx, bs, bst, bo, transpose=transpose)
    np.testing.assert_array_equal(dx.ravel().astype(np.float64), J.T @ g.ravel().astype(np.float64))


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("add", [False, True])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d" % (c[1] + c[2]))
def test_oracle_scatter_grad_is_jacobian_transpose(case, add, transpose):
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 5)
    overlap = bst[0] < bs[0] or bst[1] < bs[1]
    M, C = int(cnt[0]), shape[3]
    bshape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
    nb, ny = int(np.prod(bshape)), int(np.prod(shape))
    atomic = bool(add and overlap)
    base0 = np.zeros(shape, np.float32)
    blocks0 = np.zeros(bshape, np.float32)
    g = rng.integers(-8, 9, size=shape).astype(np.float32)
    d_blocks, d_ybase = orc.sparse_scatter_grad(g, bshape, cnt, idx, bs, bst, bo, add=add, transpose=transpose)
    # d/dybase: exact in every case (for add=False the covered pixels do not depend on ybase)
    Jy = jacobian(lambda v: orc.sparse_scatter(blocks0, cnt, idx, v.reshape(shape), bs, bst, bo, add=add,
                                               atomic=atomic, transpose=transpose), ny)
    np.testing.assert_array_equal(d_ybase.ravel().astype(np.float64), Jy.T @ g.ravel().astype(np.float64))
    # d/dblocks: the transpose of the forward map wherever the forward map is well defined.  With add=False and
    # overlapping blocks the last block in list order wins in the forward op while the reference's gradient
    # (sparse_conv_lib.py:124-130) still hands every covering block the pixel's gradient; the reference's own
    # test skips that combination (test_sparse_blocks.py:275-277), and so does this comparison.
    if add or not overlap:
        Jb = jacobian(lambda v: orc.sparse_scatter(v.reshape(bshape), cnt, idx, base0, bs, bst, bo, add=add,
                                                   atomic=atomic, transpose=transpose), nb)
        np.testing.assert_array_equal(d_blocks.ravel().astype(np.float64), Jb.T @ g.ravel().astype(np.float64))
    else:
        np.testing.assert_array_equal(d_blocks, orc.sparse_gather(g, cnt, idx, bs, bst, bo, transpose=transpose))


def test_oracle_gradients_match_finite_differences_like_the_reference_check():
    """The reference's own criterion (test_sparse_blocks.py:264-284): numeric vs analytic gradient error
    below 1e-3, on the non-overlapping geometry, for gather and for scatter with respect to (blocks, ybase)."""
    case = CASES[0]
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 9)
    x = rng.standard_normal(shape).astype(np.float32)
    w = rng.standard_normal(orc.sparse_gather(x, cnt, idx, bs, bst, bo).shape).astype(np.float32)
    f = lambda xx: float((orc.sparse_gather(xx, cnt, idx, bs, bst, bo).astype(np.float64) * w).sum())
    ana = orc.sparse_gather_grad(w, shape, cnt, idx, bs, bst, bo)
    num = np.zeros(shape, np.float64)
    eps = 1e-2
    for i in np.ndindex(*shape):
        xp, xm = x.copy(), x.copy()
        xp[i] += eps
        xm[i] -= eps
        num[i] = (f(xp) - f(xm)) / (2 * eps)
    assert np.abs(num - ana).max() < 1e-3


# ---------------------------------------------------------------------------------------------
# GPU: autograd Functions over the C ABI against the oracle's gradients
# ---------------------------------------------------------------------------------------------

GPU_CASES = CASES + [
    ((2, 40, 52, 8), (6, 6), (3, 3), (-2, -1)),
    ((1, 120, 130, 32), (27, 27), (25, 25), (-1, -1)),
    ((3, 33, 47, 5), (5, 7), (5, 7), (-2, -3)),
]
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


@pytest.mark.gpu
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("case", GPU_CASES, ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d" % (c[1] + c[2]))
def test_gather_backward_matches_oracle(case, transpose):
    import sbnet_amd
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 11)
    x = rng.standard_normal(shape).astype(np.float32)
    xd = dev(x).requires_grad_(True)
    y = sbnet_amd.sparse_gather(xd, cnt, dev(idx), bs, bst, bo, transpose=transpose)
    assert y.requires_grad
    np.testing.assert_array_equal(y.detach().cpu().numpy(), orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=transpose))
    # integer-valued cotangent: the overlapping adds are exact, so every accumulation order gives the same bits
    g = rng.integers(-8, 9, size=tuple(y.shape)).astype(np.float32)
    y.backward(dev(g))
    np.testing.assert_array_equal(xd.grad.cpu().numpy(),
                                  orc.sparse_gather_grad(g, shape, cnt, idx, bs, bst, bo, transpose=transpose))
    # real-valued cotangent: within the bar for atomic adds (1e-6 of the sum of magnitudes)
    xd.grad = None
    g = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y = sbnet_amd.sparse_gather(xd, cnt, dev(idx), bs, bst, bo, transpose=transpose)
    y.backward(dev(g))
    exp = orc.sparse_gather_grad(g, shape, cnt, idx, bs, bst, bo, transpose=transpose)
    mag = orc.sparse_gather_grad(np.abs(g), shape, cnt, idx, bs, bst, bo, transpose=transpose)
    err = np.abs(xd.grad.cpu().numpy().astype(np.float64) - exp)
    assert (err <= 1e-6 * mag).all()


@pytest.mark.gpu
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("add", [False, True])
@pytest.mark.parametrize("case", GPU_CASES, ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d" % (c[1] + c[2]))
def test_scatter_backward_matches_oracle(case, add, transpose):
    import sbnet_amd
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 13)
    overlap = bst[0] < bs[0] or bst[1] < bs[1]
    atomic = bool(add and overlap)
    M, C = int(cnt[0]), shape[3]
    bshape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
    blocks = rng.integers(-8, 9, size=bshape).astype(np.float32)
    base = rng.integers(-8, 9, size=shape).astype(np.float32)
    bd, yd = dev(blocks).requires_grad_(True), dev(base).requires_grad_(True)
    y = sbnet_amd.sparse_scatter(bd, cnt, dev(idx), yd, bs, bst, bo, add=add, atomic=atomic, transpose=transpose)
    if add or not overlap:  # with overlapping plain writes the winner is a race on the GPU
        np.testing.assert_array_equal(y.detach().cpu().numpy(),
                                      orc.sparse_scatter(blocks, cnt, idx, base, bs, bst, bo, add=add, atomic=atomic,
                                                         transpose=transpose))
    g = rng.standard_normal(shape).astype(np.float32)
    y.backward(dev(g))
    d_blocks, d_ybase = orc.sparse_scatter_grad(g, bshape, cnt, idx, bs, bst, bo, add=add, transpose=transpose)
    np.testing.assert_array_equal(bd.grad.cpu().numpy(), d_blocks)
    np.testing.assert_array_equal(yd.grad.cpu().numpy(), d_ybase)


@pytest.mark.gpu
@pytest.mark.parametrize("case", [
    # (N, H, W, C), bsize, bstride, boffset, repeated rows
    ((2, 64, 72, 32), (10, 10), (8, 8), (-1, -1), False),      # 2x2 blocks over a pixel: zeros only where no block lies
    ((1, 120, 130, 128), (27, 27), (25, 25), (-1, -1), False),  # planes split over tiles, four channel chunks
    ((2, 50, 61, 24), (7, 9), (5, 6), (2, -4), False),         # uneven everything, 6 channel vectors per pixel
    ((3, 33, 47, 5), (5, 7), (3, 4), (-2, -3), False),         # scalar channel vectors
    ((2, 40, 44, 16), (4, 4), (6, 7), (1, 0), False),          # gaps: one pass
    ((1, 30, 30, 8), (7, 7), (2, 2), (0, 0), False),           # 4x4 blocks over a pixel: cleared first, 16 passes
    ((2, 64, 72, 32), (10, 10), (8, 8), (-1, -1), True),       # a list that names blocks twice: hardware atomics
    ((1, 20, 20, 4), (1, 3), (1, 2), (0, 0), False),           # planes below 4 pixels
], ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d%s" % (c[1] + c[2] + ("_dups" if c[4] else "",)))
def test_gather_grad_entry_point(case):
    """sbnet_sparse_gather_grad (through ops.gather_backward) against the oracle's composition
    scatter(grad, zeros, add, atomic) on shuffled lists, into a tensor that holds garbage on entry."""
    from sbnet_amd import ops
    shape, bs, bst, bo, dups = case
    rng, idx, cnt = setup_case(case[:4], 23)
    if dups:
        idx = np.concatenate([idx, idx[:4]])
    rng.shuffle(idx, axis=0)
    cnt = np.array([len(idx)], np.int32)
    M, C = len(idx), shape[3]
    for transpose in (False, True):
        gshape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
        g = rng.integers(-8, 9, size=gshape).astype(np.float32)
        exp = orc.sparse_gather_grad(g, shape, cnt, idx, bs, bst, bo, transpose=transpose)
        for rep in range(2):   # (the second call finds the first one's values in the allocator's memory)
            dx = ops.gather_backward(dev(g), cnt, dev(idx), shape, bs, bst, bo, transpose)
            np.testing.assert_array_equal(dx.cpu().numpy(), exp, err_msg="transpose %s" % transpose)
            del dx
        # fewer rows than the list holds
        exp2 = orc.sparse_gather_grad(g, shape, [M - 2], idx, bs, bst, bo, transpose=transpose)
        dx = ops.gather_backward(dev(g), [M - 2], dev(idx), shape, bs, bst, bo, transpose)
        np.testing.assert_array_equal(dx.cpu().numpy(), exp2)


@pytest.mark.gpu
@pytest.mark.parametrize("case", [
    ((2, 64, 72, 32), (10, 10), (8, 8), (-1, -1)),
    ((1, 120, 130, 128), (27, 27), (25, 25), (-1, -1)),
    ((2, 50, 61, 24), (7, 9), (5, 6), (2, -4)),
    ((3, 33, 47, 5), (5, 7), (3, 4), (-2, -3)),
    ((1, 40, 40, 8), (8, 8), (4, 4), (0, 0)),                # every pixel under 2x2 blocks
], ids=lambda c: "x".join(map(str, c[0])) + "_b%dx%d_s%dx%d" % (c[1] + c[2]))
def test_gather_grad_sums_in_list_order(case):
    """With at most 2x2 blocks over a pixel and no block named twice the gradient is summed without atomics, each
    pixel as 0 + its blocks' values in list order: real-valued data (whose sums depend on the order) and signed
    zeros come out as the sequential CPU functor leaves them, bit for bit, on every call."""
    from sbnet_amd import ops
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 29, frac=0.8)
    rng.shuffle(idx, axis=0)
    M, C = len(idx), shape[3]
    for transpose in (False, True):
        gshape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
        g = (rng.standard_normal(gshape) * 10.0 ** rng.integers(-3, 4, size=gshape)).astype(np.float32)
        g[rng.random(gshape) < 0.05] = -0.0
        exp = orc.sparse_gather_grad(g, shape, cnt, idx, bs, bst, bo, transpose=transpose)
        for rep in range(2):
            dx = ops.gather_backward(dev(g), cnt, dev(idx), shape, bs, bst, bo, transpose).cpu().numpy()
            np.testing.assert_array_equal(dx.view(np.uint32), exp.view(np.uint32), err_msg="transpose %s" % transpose)


@pytest.mark.gpu
def test_chain_gather_multiply_scatter_backward():
    """x -> gather -> * w -> scatter(add) onto ybase -> sum(. * v): gradients through both Functions at once,
    against the chain rule spelled out with the oracle's pieces."""
    import sbnet_amd
    case = ((2, 40, 52, 8), (6, 6), (6, 6), (-2, -1))
    shape, bs, bst, bo = case
    rng, idx, cnt = setup_case(case, 17)
    x = rng.integers(-4, 5, size=shape).astype(np.float32)
    base = rng.integers(-4, 5, size=shape).astype(np.float32)
    w = rng.integers(-3, 4, size=(int(cnt[0]), bs[0], bs[1], shape[3])).astype(np.float32)
    v = rng.integers(-3, 4, size=shape).astype(np.float32)
    xd, yd = dev(x).requires_grad_(True), dev(base).requires_grad_(True)
    idxd = dev(idx)
    blocks = sbnet_amd.sparse_gather(xd, cnt, idxd, bs, bst, bo)
    out = sbnet_amd.sparse_scatter(blocks * dev(w), cnt, idxd, yd, bs, bst, bo, add=True)
    (out * dev(v)).sum().backward()
    d_blocks, d_ybase = orc.sparse_scatter_grad(v, w.shape, cnt, idx, bs, bst, bo, add=True)
    dx = orc.sparse_gather_grad(d_blocks * w, shape, cnt, idx, bs, bst, bo)
    np.testing.assert_array_equal(xd.grad.cpu().numpy(), dx)
    np.testing.assert_array_equal(yd.grad.cpu().numpy(), d_ybase)


@pytest.mark.gpu
def test_scatter_var_refuses_gradients():
    import sbnet_amd
    idx = torch.zeros((1, 3), dtype=torch.int16, device=DEV)
    blocks = torch.zeros((1, 2, 2, 4), device=DEV, requires_grad=True)
    base = torch.zeros((1, 4, 4, 4), device=DEV)
    with pytest.raises(NotImplementedError):
        sbnet_amd.sparse_scatter_var(blocks, [1], idx, base, (2, 2), (2, 2), (0, 0), add=False)
    with torch.no_grad():
        sbnet_amd.sparse_scatter_var(blocks, [1], idx, base, (2, 2), (2, 2), (0, 0), add=False)
