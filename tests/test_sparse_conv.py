"""Sparse convolution and the sparse ResNet bottleneck block (layers over the three block ops).

Pinned by (a) the known-answer tables of the reference's own tests (benchmark/sparse_conv_tests.py:220-268 and
437-460: an all-ones input convolved with an all-ones kernel on the active blocks counts the in-image pixels of
each window), held in tests/golden/known_answers.json, and (b) the dense twin the reference checks against
(mask_conv2d, sparse_conv_tests.py:324-349): on every output pixel of an active block the sparse result equals
the dense convolution / dense residual block.
"""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "known_answers.json")) as f:
    GOLD = json.load(f)
DEV = "cuda:0"


def covered(indices, bp, shape):
    """Boolean [N,H,W] map of the output pixels written by the active blocks (numpy, from the index list)."""
    N, H, W = shape
    idx = indices.active_block_indices.cpu().numpy()[:int(indices.bin_counts[0])]
    m = np.zeros((N, H, W), bool)
    for n, bh, bw in idx:
        h0, w0 = bh * bp.bsize_out[0], bw * bp.bsize_out[1]
        m[n, max(h0, 0):h0 + bp.bsize_out[0], max(w0, 0):w0 + bp.bsize_out[1]] = True
    return m


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("use_var", [False, True])
@pytest.mark.parametrize("case", [c for c in GOLD["pipeline"] if c["padding"] == "SAME" and
                                  c["conv_strides"] == [1, 1]], ids=lambda c: c["name"])
def test_sparse_conv2d_custom_known_answers(case, use_var, transpose):
    """SparseConv2DCustomTests._test_sparse_conv2d_custom_with_mask (sparse_conv_tests.py:400-435): the expected
    output is y_exp with the input (ones) showing through wherever no block wrote."""
    import sbnet_amd
    from sbnet_amd import sparse_conv as sc
    mask = np.asarray(case["mask"], np.float32)[None]
    H, W = mask.shape[1:]
    ksize = case["ksize"] + [1, 1]
    bp = sbnet_amd.calc_block_params([1, H, W, 1], [1] + case["bsize"] + [1], ksize, [1, 1, 1, 1], "SAME")
    assert list(bp.bstrides) == case["bstride"] and list(bp.boffset) == case["boffset"]
    ind = sc.convert_mask_to_indices_custom(torch.from_numpy(mask).to(DEV), bp, 0.0)
    x = torch.ones((1, H, W, 1), device=DEV)
    w = torch.ones(tuple(ksize), device=DEV)
    y = sc.sparse_conv2d_custom(x, w, ind, bp, [1, 1, 1, 1], use_var=use_var, transpose=transpose)
    if use_var:
        assert y.data_ptr() == x.data_ptr()
    y_exp = np.asarray(case["y_exp"], np.float32)
    y_exp = np.where(y_exp == 0, 1.0, y_exp).astype(np.float32)
    np.testing.assert_array_equal(y.cpu().numpy().reshape(y_exp.shape), y_exp)


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("kk", [1, 3, 5])
def test_sparse_conv2d_custom_matches_dense_conv(kk, transpose):
    """The reference's correctness sweep (sparse_conv_tests.py:324-359: x [10,28,28,10], kernel k in {1,3,5},
    block k+2, SAME, random mask) against the dense convolution on the pixels the blocks write; the
    reference's tolerance is rtol 1e-2 / atol 0.1, fp32 convolution algorithms agree far better."""
    import sbnet_amd
    from sbnet_amd import sparse_conv as sc
    rng = np.random.RandomState(0)
    xsize = [10, 28, 28, 10]
    x = rng.uniform(-1, 1, xsize).astype(np.float32)
    w = rng.uniform(-1, 1, [kk, kk, 10, 10]).astype(np.float32)
    mask = (rng.uniform(-5, 1, xsize[:-1]) > 0).astype(np.float32)
    bp = sbnet_amd.calc_block_params(xsize, [1, kk + 2, kk + 2, 1], [kk, kk, 10, 10], [1, 1, 1, 1], "SAME")
    xd, wd, md = (torch.from_numpy(a).to(DEV) for a in (x, w, mask))
    ind = sc.convert_mask_to_indices_custom(md, bp, 0.0)
    y = sc.sparse_conv2d_custom(xd, wd, ind, bp, [1, 1, 1, 1], transpose=transpose).cpu().numpy()
    dense = sc.mask_conv2d(xd, wd, torch.ones_like(md), [1, 1, 1, 1], "SAME").cpu().numpy()
    cov = covered(ind, bp, xsize[:3])
    assert cov.any() and not cov.all()
    np.testing.assert_allclose(y[cov], dense[cov], rtol=1e-4, atol=1e-4)
    np.testing.assert_array_equal(y[~cov], x[~cov])   # untouched pixels keep the input
    # (calc_block_params, as in the reference, can leave the last output row/column without a block: 28 pixels,
    # 5x5 blocks at stride 3 give 9 blocks that write outputs 0..26; coverage is therefore not asserted)


@pytest.mark.parametrize("data_format", ["NHWC", "NCHW"])
@pytest.mark.parametrize("use_var", [False, True])
def test_sparse_res_block_matches_dense_on_active_blocks(data_format, use_var):
    """y = x + F(x) on the active blocks equals the dense residual block there, and y = x elsewhere
    (geometry of SparseResBlockGradientTests, sparse_res_block_tests.py:255-268, in inference mode so that
    batch norm uses the same statistics on both sides)."""
    import sbnet_amd
    from sbnet_amd import sparse_conv as sc
    rnd = np.random.RandomState(0)
    mask = (rnd.uniform(0, 1, [3, 9, 9]) > 0.5).astype(np.float32)
    mask[1] = 0.0
    mask[1, 4, 4] = 1.0
    ch = 8
    xval = (rnd.uniform(-0.1, 0.1, [3, 9, 9, ch]) + 1.0).astype(np.float32)
    ksize_list = [[1, 1, ch, ch // 4], [3, 3, ch // 4, ch // 4], [1, 1, ch // 4, ch]]
    bp = sbnet_amd.calc_block_params_res_block(list(xval.shape), [1, 5, 5, 1], ksize_list, [1, 1, 1, 1], "SAME")
    params = sc.BottleneckParams(ksize_list, DEV, seed=3)
    x = torch.from_numpy(xval).to(DEV)
    ind = sc.convert_mask_to_indices_custom(torch.from_numpy(mask).to(DEV), bp, 0.0)
    with torch.no_grad():
        dense = sc.res_block_bottleneck(x, params, [1, 1, 1, 1], is_training=False).cpu().numpy()
        y = sc.sparse_res_block_bottleneck(x.clone(), params, ind, bp, [1, 1, 1, 1], is_training=False,
                                           data_format=data_format, use_var=use_var).cpu().numpy()
    cov = covered(ind, bp, xval.shape[:3])
    assert cov.any() and not cov.all()
    np.testing.assert_allclose(y[cov], dense[cov], rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(y[~cov], xval[~cov])


def test_sparse_res_block_gradients_match_dense_where_blocks_are_isolated():
    """Gradients through gather -> BN/ReLU/conv x3 -> scatter-add, against autograd of the dense block.  With
    one active block in the middle of the image and a loss restricted to that block's output, the two graphs
    compute the same function of x and of the weights."""
    import sbnet_amd
    from sbnet_amd import sparse_conv as sc
    rnd = np.random.RandomState(1)
    ch = 8
    xval = (rnd.uniform(-0.5, 0.5, [1, 15, 15, ch])).astype(np.float32)
    mask = np.zeros([1, 15, 15], np.float32)
    mask[0, 7, 7] = 1.0
    ksize_list = [[1, 1, ch, ch // 4], [3, 3, ch // 4, ch // 4], [1, 1, ch // 4, ch]]
    bp = sbnet_amd.calc_block_params_res_block(list(xval.shape), [1, 5, 5, 1], ksize_list, [1, 1, 1, 1], "SAME")
    ind = sc.convert_mask_to_indices_custom(torch.from_numpy(mask).to(DEV), bp, 0.0)
    assert int(ind.bin_counts[0]) == 1
    cov = torch.from_numpy(covered(ind, bp, xval.shape[:3])).to(DEV)
    weight = torch.from_numpy(rnd.uniform(-1, 1, xval.shape).astype(np.float32)).to(DEV) * cov[..., None]
    grads = []
    for sparse in (False, True):
        params = sc.BottleneckParams(ksize_list, DEV, seed=5)
        x = torch.from_numpy(xval).to(DEV).requires_grad_(True)
        if sparse:
            y = sc.sparse_res_block_bottleneck(x, params, ind, bp, [1, 1, 1, 1], is_training=False)
        else:
            y = sc.res_block_bottleneck(x, params, [1, 1, 1, 1], is_training=False)
        (y * weight).sum().backward()
        grads.append([x.grad.cpu().numpy()] + [p.grad.cpu().numpy() for p in params.parameters()])
    for a, b in zip(*grads):
        np.testing.assert_allclose(b, a, rtol=1e-4, atol=1e-5)


def test_timer_twins_measure_device_time():
    """hip_timer_start_op / hip_timer_end_op (CudaTimerStart / CudaTimerEnd, sparse_gather.cc:390-469):
    milliseconds of device time between the two records."""
    from sbnet_amd import sparse_conv as sc
    a = torch.empty(64 << 20, device=DEV)
    a.zero_()
    torch.cuda.synchronize()
    t0 = sc.hip_timer_start_op()
    for _ in range(20):
        a.add_(1.0)
    dt = sc.hip_timer_end_op(t0)
    ref0, ref1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ref0.record()
    for _ in range(20):
        a.add_(1.0)
    ref1.record()
    ref1.synchronize()
    ref = ref0.elapsed_time(ref1)
    assert isinstance(dt, float) and dt > 0.0
    assert 0.5 * ref < dt < 2.0 * ref + 0.5


def test_benchmark_run_one_dense_and_sparse():
    """run_one of the top-left-mask benchmark (sparse_conv_perf.py:208-262) on a small stage: times are positive
    and the block sparsity follows from the mask: a top-left square of density 0.25 on 40x60 with 5x5 input
    blocks (3x3 outputs) activates ceil-covered blocks only."""
    from sbnet_amd import benchmark_topleft as bt
    xsize, ksize = [1, 40, 60, 16], [3, 3, 16, 4]
    dense = bt.run_one(None, bt.TestConfig(xsize, ksize, None, [1, 1, 1, 1], "SAME", False, None, None),
                       res_block=True, n_warmup=1, n_run=1, n_repeat=2)
    assert dense.avg_time > 0 and dense.block_sparsity == 0.0
    mask = bt.generate_top_left_mask(xsize, 0.75)
    assert mask.shape == (1, 40, 60) and mask.sum() == 20 * 30 and mask[0, :20, :30].all()
    for res_block in (False, True):
        k = ksize if res_block else [3, 3, 16, 16]
        r = bt.run_one(mask, bt.TestConfig(xsize, k, [1, 5, 5, 1], [1, 1, 1, 1], "SAME", True, bt.TOL, bt.AVGPOOL),
                       res_block=res_block, n_warmup=1, n_run=1, n_repeat=2)
        assert r.avg_time > 0
        # blocks start at -1 + 3*b and are active when more than 5 % of 25 pixels are set: rows b <= 6 (start 17,
        # 3 rows inside), columns b <= 10 (start 29: 1 column inside, 5/25 > 0.05): 7 x 11 of the 13 x 20 blocks that
        # calc_block_params lays over 40 x 60
        assert abs(r.block_sparsity - (1.0 - 7 * 11 / (13 * 20.0))) < 1e-6


@pytest.mark.parametrize("data_format", ["NHWC", "NCHW"])
def test_sparse_res_block_in_a_hip_graph_replays_identically(data_format):
    """The three block ops enqueue on the caller's stream and allocate nothing of their own, so a whole sparse
    residual block can be captured into a HIP graph.  Every replay, with eager work and synchronisation in
    between, must reproduce the eager result for the input present at replay time."""
    import sbnet_amd
    from sbnet_amd import sparse_conv as sc
    rnd = np.random.RandomState(2)
    ch = 16
    shape = [2, 30, 40, ch]
    mask = (rnd.uniform(0, 1, shape[:3]) > 0.8).astype(np.float32)
    ksize_list = [[1, 1, ch, ch // 4], [3, 3, ch // 4, ch // 4], [1, 1, ch // 4, ch]]
    bp = sbnet_amd.calc_block_params_res_block(shape, [1, 7, 7, 1], ksize_list, [1, 1, 1, 1], "SAME")
    params = sc.BottleneckParams(ksize_list, DEV, seed=7)
    ind = sc.convert_mask_to_indices_custom(torch.from_numpy(mask).to(DEV), bp, 0.0)
    x_static = torch.zeros(shape, device=DEV)

    def layer():
        return sc.sparse_res_block_bottleneck(x_static, params, ind, bp, [1, 1, 1, 1], is_training=False,
                                              data_format=data_format)

    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            layer()
            layer()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = layer()
        for rep in range(4):
            xval = torch.from_numpy(rnd.uniform(-1, 1, shape).astype(np.float32)).to(DEV)
            x_static.copy_(xval)
            graph.replay()
            torch.cuda.synchronize()
            got = y_static.clone()
            exp = sc.sparse_res_block_bottleneck(xval, params, ind, bp, [1, 1, 1, 1], is_training=False,
                                                 data_format=data_format)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(got.cpu().numpy(), exp.cpu().numpy())


# ---------------------------------------------------------------------------------------------
# The reference's index-list interface (convert_mask_to_block_indices / upsample_indices / sparse_conv2d /
# sparse_conv2d_matmul), pinned by the vectors its own tests hold
# ---------------------------------------------------------------------------------------------

# benchmark/sparse_conv_tests.py:68-100: two 3x3 windows at (0,1,2) and (0,2,0), stride 1
UPSAMPLE_IND = [[0, 1, 2], [0, 2, 0]]
UPSAMPLE_EXP = [[0, 1, 2], [0, 1, 3], [0, 1, 4], [0, 2, 2], [0, 2, 3], [0, 2, 4], [0, 3, 2], [0, 3, 3], [0, 3, 4],
                [0, 2, 0], [0, 2, 1], [0, 2, 2], [0, 3, 0], [0, 3, 1], [0, 3, 2], [0, 4, 0], [0, 4, 1], [0, 4, 2]]


def test_upsample_indices_known_answer():
    from sbnet_amd import sparse_conv as sc
    ind = torch.tensor(UPSAMPLE_IND, dtype=torch.int32, device=DEV)
    up = sc.upsample_indices(ind, [1, 3, 3, 1], [1, 1, 1, 1])
    assert tuple(up.shape) == (2, 3, 3, 3) and up.dtype == torch.int32
    np.testing.assert_array_equal(up.cpu().numpy().reshape(-1, 3), np.asarray(UPSAMPLE_EXP, np.int32))
    # a pooling step of 2 moves the windows, not their pixels (sparse_conv_lib.py:266-275)
    up2 = sc.upsample_indices(ind, [1, 2, 3, 1], [1, 2, 2, 1]).cpu().numpy()
    assert up2.shape == (2, 2, 3, 3)
    np.testing.assert_array_equal(up2[0, :, :, 1:], [[[2, 4], [2, 5], [2, 6]], [[3, 4], [3, 5], [3, 6]]])


@pytest.mark.parametrize("padding,y_exp", [
    # benchmark/sparse_conv_tests.py:107-148 (VALID) and 150-193 (SAME): the same two hand-written rectangles
    ("VALID", [[0, 0, 0], [0, 0, 9], [9, 0, 0]]),
    ("SAME", [[0, 0, 0, 0, 0], [0, 0, 9, 0, 0], [6, 0, 0, 0, 0], [0, 0, 0, 0, 0], [0, 0, 0, 0, 0]]),
])
def test_sparse_conv2d_hand_written_rectangles(padding, y_exp):
    from sbnet_amd import sparse_conv as sc
    ind_blk = torch.tensor(UPSAMPLE_EXP, dtype=torch.int32, device=DEV).view(2, 3, 3, 3)
    x = torch.ones((1, 5, 5, 1), device=DEV)
    w = torch.ones((3, 3, 1, 1), device=DEV)
    y = sc.sparse_conv2d(x, w, ind_blk, [1, 1, 1, 1], padding)
    y_exp = np.asarray(y_exp, np.float32)
    assert y.numel() == y_exp.size
    np.testing.assert_array_equal(y.cpu().numpy().reshape(y_exp.shape), y_exp)


@pytest.mark.parametrize("case", GOLD["pipeline"], ids=lambda c: c["name"])
def test_sparse_conv2d_with_mask_known_answers(case):
    """SparseConv2DTests._test_sparse_conv2d_with_mask (sparse_conv_tests.py:195-321): mask -> block indices ->
    sparse_conv2d of ones with a kernel of ones, all five tables, stride-2 and VALID ones included."""
    from sbnet_amd import sparse_conv as sc
    mask = torch.tensor(case["mask"], dtype=torch.float32, device=DEV)[None]
    bsize, ksize = [1] + case["bsize"] + [1], case["ksize"] + [1, 1]
    strides = [1] + case["conv_strides"] + [1]
    ind_blk = sc.convert_mask_to_block_indices(mask, bsize, ksize, strides, case["padding"], 0.0)
    assert ind_blk.dtype == torch.int32 and tuple(ind_blk.shape[1:]) == (case["bsize"][0], case["bsize"][1], 3)
    x = torch.ones((1, mask.shape[1], mask.shape[2], 1), device=DEV)
    w = torch.ones(tuple(ksize), device=DEV)
    y = sc.sparse_conv2d(x, w, ind_blk, strides, case["padding"])
    y_exp = np.asarray(case["y_exp"], np.float32)
    assert y.numel() == y_exp.size
    np.testing.assert_array_equal(y.cpu().numpy().reshape(y_exp.shape), y_exp)


def _random_problem(kk, cout=10):
    rng = np.random.RandomState(0)
    xsize = [10, 28, 28, 10]
    x = rng.uniform(-1, 1, xsize).astype(np.float32)
    w = rng.uniform(-1, 1, [kk, kk, 10, cout]).astype(np.float32)
    mask = (rng.uniform(-5, 1, xsize[:-1]) > 0).astype(np.float32)
    return (torch.from_numpy(a).to(DEV) for a in (x, w, mask))


def _compare_on_active_outputs(y_act, x, w, mask, strides, padding):
    """The reference compares where the max-pooled mask is set (sparse_conv_tests.py:336-349) with rtol 1e-2 /
    atol 0.1; fp32 convolutions agree far better, and outside the active rectangles the sparse result is 0."""
    from sbnet_amd import sparse_conv as sc
    y_exp = sc.mask_conv2d(x, w, mask, strides, padding)
    kh, kw = int(w.shape[0]), int(w.shape[1])
    m = sc._pool_same_or_valid(mask[:, None], (kh, kw), (strides[1], strides[2]), padding)[:, 0] > 0
    assert y_act.shape == y_exp.shape and int(m.sum()) > 0
    torch.testing.assert_close(y_act[m], y_exp[m], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("ss", [1, 2])
@pytest.mark.parametrize("padding", ["SAME", "VALID"])
@pytest.mark.parametrize("kk", [1, 3, 5])
def test_sparse_conv2d_matches_dense_conv(kk, padding, ss):
    """SparseConv2DTests.test_sparse_conv2d_correctness (sparse_conv_tests.py:324-359): x [10,28,28,10], kernel
    k in {1,3,5}, blocks of k+2, both paddings, strides 1 and 2."""
    from sbnet_amd import sparse_conv as sc
    x, w, mask = _random_problem(kk)
    strides = [1, ss, ss, 1]
    if (kk + 2 - kk) % ss != 0:
        with pytest.raises(AssertionError):   # `stride` must divide `bsize` - `ksize`
            sc.convert_mask_to_block_indices(mask, [1, kk + 2, kk + 2, 1], [kk, kk, 10, 10], strides, padding, 0.0)
        return
    ind_blk = sc.convert_mask_to_block_indices(mask, [1, kk + 2, kk + 2, 1], [kk, kk, 10, 10], strides, padding, 0.0)
    y = sc.sparse_conv2d(x, w, ind_blk, strides, padding)
    _compare_on_active_outputs(y, x, w, mask, strides, padding)


@pytest.mark.parametrize("padding", ["SAME", "VALID"])
@pytest.mark.parametrize("kk", [1, 3, 5])
def test_sparse_conv2d_matmul_matches_dense_conv(kk, padding):
    """SparseConv2DTests.test_sparse_conv2d_matmul_correctness (sparse_conv_tests.py:361-397): blocks of the
    kernel's size, one output pixel each."""
    from sbnet_amd import sparse_conv as sc
    x, w, mask = _random_problem(kk, cout=7)
    strides = [1, 1, 1, 1]
    ind_blk = sc.convert_mask_to_block_indices(mask, [1, kk, kk, 1], [kk, kk, 10, 7], strides, padding, 0.0)
    y = sc.sparse_conv2d_matmul(x, w, ind_blk, strides, padding)
    _compare_on_active_outputs(y, x, w, mask, strides, padding)
    # on these rectangles the two index-list convolutions compute the same thing
    y2 = sc.sparse_conv2d(x, w, ind_blk, strides, padding)
    torch.testing.assert_close(y, y2, rtol=1e-4, atol=1e-4)
    with pytest.raises(ValueError):
        sc.sparse_conv2d_matmul(x, w, ind_blk, [1, 2, 2, 1], padding)


def test_index_list_interface_corner_cases():
    from sbnet_amd import sparse_conv as sc
    x, w, mask = _random_problem(3)
    bsize, ksize, strides = [1, 5, 5, 1], [3, 3, 10, 10], [1, 1, 1, 1]
    # no active block: an empty list and a zero result of the convolution's shape
    none = sc.convert_mask_to_block_indices(torch.zeros_like(mask), bsize, ksize, strides, "SAME", 0.0)
    assert tuple(none.shape) == (0, 5, 5, 3)
    y = sc.sparse_conv2d(x, w, none, strides, "SAME")
    assert tuple(y.shape) == (10, 28, 28, 10) and float(y.abs().max()) == 0.0
    # a negative tolerance: the zeros of the padding count, so every block is active (tf.nn.max_pool over tf.pad)
    every = sc.convert_mask_to_indices(torch.zeros_like(mask), bsize, ksize, strides, "SAME", -0.5)
    assert every.shape[0] == 10 * 10 * 10   # 28 + 2 padded to 32 -> (32 - 5) // 3 + 1 = 10 blocks per axis
    # The block grid is the custom op's (same windows, same order) with one more row and column of blocks: the
    # index-list path pads the far side from the padded extent (sparse_conv_lib.py:170-174: 30 -> 32 rows, 10
    # blocks), calc_block_params from the unpadded one (:370-374: 31 rows, 9 blocks).
    import sbnet_amd
    bp = sbnet_amd.calc_block_params([10, 28, 28, 10], bsize, ksize, strides, "SAME")
    assert list(bp.bcount) == [9, 9]
    ind = sc.convert_mask_to_indices_custom(mask, bp, 0.0)
    lst = sc.convert_mask_to_indices(mask, bsize, ksize, strides, "SAME", 0.0).cpu().numpy()
    assert lst[:, 1].max() == 9 and lst[:, 2].max() == 9
    common = lst[(lst[:, 1] < 9) & (lst[:, 2] < 9)]
    np.testing.assert_array_equal(common,
                                  ind.active_block_indices[:int(ind.bin_counts[0])].cpu().numpy().astype(np.int32))
    lst = torch.from_numpy(lst).to(DEV)
    # rectangles must be rectangles
    bad = sc.upsample_indices(lst[:4], bsize, [1, 3, 3, 1]).clone()
    bad[1, 2, 2, 1] += 1
    with pytest.raises(ValueError):
        sc.sparse_conv2d(x, w, bad, strides, "SAME")


def test_sparse_conv2d_gradients_match_the_masked_dense_convolution():
    """Loss restricted to the active outputs: d/dw and d/dx through gather -> conv -> scatter equal those of the
    dense convolution (the gradients of the block ops are the reference's compositions, sparse_conv_lib.py:80-147)."""
    from sbnet_amd import sparse_conv as sc
    x, w, mask = _random_problem(3)
    strides, padding = [1, 1, 1, 1], "SAME"
    ind_blk = sc.convert_mask_to_block_indices(mask, [1, 5, 5, 1], [3, 3, 10, 10], strides, padding, 0.0)
    g = torch.Generator(device=DEV).manual_seed(3)
    probe = torch.randn((10, 28, 28, 10), generator=g, device=DEV)
    xs, ws = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y = sc.sparse_conv2d(xs, ws, ind_blk, strides, padding)
    # outputs a rectangle writes: the interior left after a VALID 3x3 convolution of each 5x5 block
    out_mask = torch.zeros((10, 28, 28), device=DEV)
    o = ind_blk[:, 0, 0, :].long()
    for dh in range(3):
        for dw in range(3):
            hh, ww = o[:, 1] + dh, o[:, 2] + dw
            ok = (hh < 28) & (ww < 28)
            out_mask[o[ok, 0], hh[ok], ww[ok]] = 1.0
    (y * probe).sum().backward()
    xd, wd = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    yd = sc._conv_same_or_valid(xd.permute(0, 3, 1, 2), sc._hwio_to_oihw(wd), (1, 1), padding).permute(0, 2, 3, 1)
    (yd * probe * out_mask[..., None]).sum().backward()
    torch.testing.assert_close(y.detach(), (yd * out_mask[..., None]).detach(), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(ws.grad, wd.grad, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(xs.grad, xd.grad, rtol=1e-4, atol=1e-4)


def test_readme_attribute_spelling_and_sample():
    """The reference's README.md:53-107 and sample.py:42-43 pass the block parameters as `bsize=`, `bstride=`,
    `boffset=` (and the block count second); the op wrappers take both spellings, and the sample layer written that
    way reproduces the dense convolution on the blocks it writes."""
    import sbnet_amd
    from sbnet_amd import sample
    rng = np.random.default_rng(4)
    mask = torch.from_numpy((rng.random((2, 20, 20, 1)) < 0.2).astype(np.float32)).to(DEV)
    x = torch.from_numpy(rng.standard_normal((2, 20, 20, 8)).astype(np.float32)).to(DEV)
    a = sbnet_amd.reduce_mask(mask, [5, 5], [6, 6], [4, 4], [-1, -1], 0.5)
    b = sbnet_amd.reduce_mask(mask, [5, 5], bsize=[6, 6], boffset=[-1, -1], bstride=[4, 4], tol=0.5)
    assert int(a.bin_counts[0]) == int(b.bin_counts[0]) > 0
    assert torch.equal(a.active_block_indices[:int(a.bin_counts[0])], b.active_block_indices[:int(b.bin_counts[0])])
    kw = dict(bsize=[6, 6], boffset=[-1, -1], bstride=[4, 4])
    g1 = sbnet_amd.sparse_gather(x, a.bin_counts, a.active_block_indices, [6, 6], [4, 4], [-1, -1], transpose=True)
    g2 = sbnet_amd.sparse_gather(x, a.bin_counts, a.active_block_indices, transpose=True, **kw)
    assert torch.equal(g1, g2)
    y1 = sbnet_amd.sparse_scatter(g1, a.bin_counts, a.active_block_indices, x, [6, 6], [4, 4], [-1, -1], add=True,
                                  atomic=True, transpose=True)
    y2 = sbnet_amd.sparse_scatter(g1, a.bin_counts, a.active_block_indices, x, add=True, atomic=True, transpose=True,
                                  **kw)
    assert torch.equal(y1, y2)
    with pytest.raises(TypeError):
        sbnet_amd.sparse_gather(x, a.bin_counts, a.active_block_indices, [6, 6], [4, 4], [-1, -1], bsize=[6, 6])
    with pytest.raises(TypeError):
        sbnet_amd.sparse_gather(x, a.bin_counts, a.active_block_indices, bsize=[6, 6], bstride=[4, 4])
    with pytest.raises(TypeError):
        sbnet_amd.sparse_scatter(g1, a.bin_counts, a.active_block_indices, x, **kw)   # add has no default
    y = sample.main(seed=1, device=DEV)
    assert tuple(y.shape) == (4, 254, 254, 64)
