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
