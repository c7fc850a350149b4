"""Pins the CPU oracle (oracle/sbnet_oracle.c) before anything is compared against it.

Checks, none of which re-type the oracle's own loops:
  * the reference tests' hand-written masks and known-answer tables (tests/golden/known_answers.json);
  * library twins: torch max_pool2d / avg_pool2d on explicitly padded masks, torch fold for
    overlapping scatter-add;
  * numpy slicing of the zero-padded tensor (tests/closed_forms.py);
  * invariants: transposed == transpose(untransposed), scatter(gather(x)) restores x on covered pixels,
    the zero-count special case, summation-order sensitivity of avg pooling.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from closed_forms import box_sum_valid, np_gather, np_reduce_mask, np_scatter
from oracle import sbnet_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "known_answers.json")) as f:
    GOLD = json.load(f)


def active(res):
    idx, cnt = res
    return idx[:int(cnt[0])]


# ---------------------------------------------------------------------------------------------
# golden vectors held by the reference's own tests
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("case", GOLD["reduce_mask"], ids=lambda c: c["name"])
def test_reduce_mask_golden(case):
    mask = np.asarray(case["mask"], np.float32)[None, :, :, None]
    got = active(orc.reduce_mask(mask, case["bcount"], case["bsize"], case["bstride"], case["boffset"],
                                 case["tol"], case["avgpool"]))
    assert got.tolist() == case["expected_indices"]


@pytest.mark.parametrize("case", GOLD["gather_arange"], ids=lambda c: c["name"])
def test_gather_arange_golden(case):
    H, W = case["shape"]
    x = np.arange(H * W, dtype=np.float32).reshape(1, H, W, 1)
    idx = np.asarray(case["indices"], np.int16)
    y = orc.sparse_gather(x, [len(idx)], idx, case["bsize"], case["bstride"], case["boffset"])
    assert y.reshape(len(idx), -1).tolist() == case["expected_blocks"]


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("case", GOLD["pipeline"], ids=lambda c: c["name"])
def test_pipeline_known_answers(case, transpose):
    """mask -> reduce_mask -> gather -> all-ones VALID conv -> scatter equals the reference tests' y_exp."""
    mask = np.asarray(case["mask"], np.float32)[None, :, :, None]
    x = np.ones_like(mask)
    idx, cnt = orc.reduce_mask(mask, case["bcount"], case["bsize"], case["bstride"], case["boffset"], 0.0)
    p = orc.sparse_gather(x, cnt, idx, case["bsize"], case["bstride"], case["boffset"], transpose=transpose)
    p_nhwc = p.transpose(0, 2, 3, 1) if transpose else p
    q = box_sum_valid(p_nhwc, case["ksize"][0], case["ksize"][1], *case["conv_strides"])
    assert list(q.shape[1:3]) == case["bsize_out"]
    if transpose:
        q = np.ascontiguousarray(q.transpose(0, 3, 1, 2))
    y_exp = np.asarray(case["y_exp"], np.float32)[None, :, :, None]
    y = orc.sparse_scatter(q, cnt, idx, np.zeros_like(y_exp), case["bsize_out"], case.get("s_bstride", case["bstride"]),
                           [0, 0], add=False, transpose=transpose)
    np.testing.assert_array_equal(y, y_exp)


def test_config1_digests():
    from golden.make_fixtures import config1_inputs, sha
    c = GOLD["config1"]
    x, mask = config1_inputs(c["seed"])
    assert sha(x) == c["x_sha256"] and sha(mask) == c["mask_sha256"]
    idx, cnt = orc.reduce_mask(mask, c["bcount"], c["bsize"], c["bstride"], c["boffset"], c["tol"], c["avgpool"])
    assert active((idx, cnt)).tolist() == c["expected_indices"]
    g = orc.sparse_gather(x, cnt, idx, c["bsize"], c["bstride"], c["boffset"])
    gt = orc.sparse_gather(x, cnt, idx, c["bsize"], c["bstride"], c["boffset"], transpose=True)
    y = orc.sparse_scatter(g, cnt, idx, np.zeros_like(x), c["bsize"], c["bstride"], c["boffset"], add=False)
    assert sha(g) == c["gather_sha256"] and sha(gt) == c["gather_t_sha256"] and sha(y) == c["scatter_sha256"]


# ---------------------------------------------------------------------------------------------
# reduce_mask against library twins and closed forms
# ---------------------------------------------------------------------------------------------

# (H, W), bsize, bstride, boffset, N : the shape menu of the reference's integration test
# (sbnet_ops/tests/test_sparse_blocks.py:345-449): overlaps, gaps, uneven offsets, N > 1
GEOMS = [
    ((5, 5), (3, 3), (1, 1), (-1, -2), 1),
    ((2, 3), (2, 3), (3, 4), (-1, -2), 1),
    ((8, 10), (3, 4), (3, 4), (-1, -2), 3),
    ((8, 10), (3, 4), (4, 5), (-1, -2), 1),
    ((5, 5), (3, 2), (3, 2), (-1, -2), 1),
    ((5, 3), (2, 3), (2, 3), (0, 0), 7),
    ((3, 3), (2, 2), (1, 1), (0, 0), 1),
    ((3, 3), (1, 1), (2, 2), (-1, -2), 1),
    ((13, 12), (2, 3), (1, 2), (0, 0), 2),
    ((40, 60), (3, 4), (2, 3), (-1, -2), 2),
    ((64, 64), (10, 10), (8, 8), (-1, -1), 1),
    ((70, 50), (18, 18), (16, 16), (-1, -1), 2),
    ((100, 100), (27, 27), (25, 25), (-1, -1), 1),
]


def bcount_covering(H, W, bstride, boffset):
    return [1 + (H - boffset[0] - 1) // bstride[0], 1 + (W - boffset[1] - 1) // bstride[1]]


@pytest.mark.parametrize("geom", GEOMS, ids=str)
def test_reduce_mask_max_vs_torch_maxpool(geom):
    (H, W), bs, bst, bo, N = geom
    rng = np.random.default_rng(7)
    bc = bcount_covering(H, W, bst, bo)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    tol = float(np.percentile(mask, 70))
    hend = bo[0] + bst[0] * (bc[0] - 1) + bs[0]
    wend = bo[1] + bst[1] * (bc[1] - 1) + bs[1]
    t = torch.from_numpy(mask).permute(0, 3, 1, 2)
    t = F.pad(t, (max(0, -bo[1]), max(0, wend - W), max(0, -bo[0]), max(0, hend - H)), value=float("-inf"))
    pooled = F.max_pool2d(t, kernel_size=tuple(bs), stride=tuple(bst))[:, 0]
    assert list(pooled.shape[1:]) == bc
    exp = torch.nonzero(pooled > tol).numpy().astype(np.int16)
    got = active(orc.reduce_mask(mask, bc, bs, bst, bo, tol, False))
    if len(exp) == 0:
        assert got.tolist() == [[0, 0, 0]]
    else:
        np.testing.assert_array_equal(got, exp)
    np.testing.assert_array_equal(np_reduce_mask(mask, bc, bs, bst, bo, tol, False), exp)


@pytest.mark.parametrize("geom", GEOMS, ids=str)
def test_reduce_mask_avg_vs_torch_avgpool(geom):
    """Binary masks: every summation order gives the exact integer, so torch's pooling is a twin as
    long as no block sits on the threshold (tol is chosen between two attainable averages)."""
    (H, W), bs, bst, bo, N = geom
    rng = np.random.default_rng(11)
    bc = bcount_covering(H, W, bst, bo)
    mask = (rng.random((N, H, W, 1)) < 0.4).astype(np.float32)
    area = bs[0] * bs[1]
    tol = (max(1, area // 3) - 0.5) / area
    hend = bo[0] + bst[0] * (bc[0] - 1) + bs[0]
    wend = bo[1] + bst[1] * (bc[1] - 1) + bs[1]
    t = torch.from_numpy(mask).permute(0, 3, 1, 2).double()
    t = F.pad(t, (max(0, -bo[1]), max(0, wend - W), max(0, -bo[0]), max(0, hend - H)), value=0.0)
    pooled = F.avg_pool2d(t, kernel_size=tuple(bs), stride=tuple(bst))[:, 0]
    assert (pooled - tol).abs().min() > 1e-4
    exp = torch.nonzero(pooled > tol).numpy().astype(np.int16)
    got = active(orc.reduce_mask(mask, bc, bs, bst, bo, tol, True))
    if len(exp) == 0:
        assert got.tolist() == [[0, 0, 0]]
    else:
        np.testing.assert_array_equal(got, exp)
    np.testing.assert_array_equal(np_reduce_mask(mask, bc, bs, bst, bo, tol, True), exp)


def test_reduce_mask_avg_divides_by_full_block_area():
    """A clipped corner block still divides by bsize[0]*bsize[1] (reduce_mask.cc:87-88)."""
    mask = np.ones((1, 4, 4, 1), np.float32)
    # block (0,0) at offset -1 sees 2x2 = 4 of its 9 pixels: average 4/9
    got = active(orc.reduce_mask(mask, [1, 1], [3, 3], [3, 3], [-1, -1], 0.45, True))
    assert got.tolist() == [[0, 0, 0]]
    idx, cnt = orc.reduce_mask(mask, [2, 2], [3, 3], [2, 2], [-1, -1], 0.45, True)
    # blocks: (0,0) 4/9 no; (0,1) rows -1..1 cols 1..3 -> 2x3=6/9 yes; (1,0) yes; (1,1) 9/9 yes
    assert active((idx, cnt)).tolist() == [[0, 0, 1], [0, 1, 0], [0, 1, 1]]


def test_reduce_mask_strict_greater_and_zero_count():
    mask = np.full((2, 4, 4, 1), 0.5, np.float32)
    idx, cnt = orc.reduce_mask(mask, [2, 2], [2, 2], [2, 2], [0, 0], 0.5, False)
    # nothing is strictly greater: count 1 and the triple (0,0,0) (test_sparse_blocks.py:303-306)
    assert int(cnt[0]) == 1 and idx[0].tolist() == [0, 0, 0]
    idx, cnt = orc.reduce_mask(mask, [2, 2], [2, 2], [2, 2], [0, 0], 0.5, True)
    assert int(cnt[0]) == 1 and idx[0].tolist() == [0, 0, 0]
    idx, cnt = orc.reduce_mask(mask, [2, 2], [2, 2], [2, 2], [0, 0], 0.49, True)
    assert int(cnt[0]) == 8


def test_reduce_mask_avg_sums_in_row_major_order():
    """fp32 addition order matters; the oracle must use the CPU functor's row-major order."""
    vals = np.array([[1e8, 1.0, -1e8], [1.0, 1.0, 1.0]], np.float32)
    mask = vals.reshape(1, 2, 3, 1)
    s = np.float32(0)
    for v in vals.reshape(-1):
        s = np.float32(s + v)
    assert s == np.float32(3.0)  # (1e8 + 1) rounds to 1e8, so the first 1.0 is lost
    assert float(np.sum(vals.astype(np.float64))) == 4.0
    tol_between = 3.5 / 6.0
    assert int(orc.reduce_mask(mask, [1, 1], [2, 3], [2, 3], [0, 0], tol_between, True)[1][0]) == 1
    assert active(orc.reduce_mask(mask, [1, 1], [2, 3], [2, 3], [0, 0], tol_between, True)).tolist() == [[0, 0, 0]]
    # with a threshold just under 3/6 the block is genuinely active
    idx, cnt = orc.reduce_mask(np.concatenate([mask, mask]), [1, 1], [2, 3], [2, 3], [0, 0], 2.9 / 6.0, True)
    assert active((idx, cnt)).tolist() == [[0, 0, 0], [1, 0, 0]]
    idx, cnt = orc.reduce_mask(np.concatenate([mask * 0, mask]), [1, 1], [2, 3], [2, 3], [0, 0], tol_between, True)
    assert active((idx, cnt)).tolist() == [[0, 0, 0]] and int(cnt[0]) == 1  # fix-up, not a real hit


# ---------------------------------------------------------------------------------------------
# gather / scatter against numpy slicing and torch fold
# ---------------------------------------------------------------------------------------------

CHANNELS = [1, 2, 3, 7, 16]


@pytest.mark.parametrize("C", CHANNELS)
@pytest.mark.parametrize("geom", GEOMS[:10], ids=str)
def test_gather_vs_numpy_slices(geom, C):
    (H, W), bs, bst, bo, N = geom
    rng = np.random.default_rng(3)
    bc = bcount_covering(H, W, bst, bo)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    idx, cnt = orc.reduce_mask(mask, bc, bs, bst, bo, float(np.percentile(mask, 50)), False)
    a = active((idx, cnt))
    y = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=False)
    yt = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=True)
    np.testing.assert_array_equal(y, np_gather(x, a, bs, bst, bo, False))
    np.testing.assert_array_equal(yt, y.transpose(0, 3, 1, 2))
    np.testing.assert_array_equal(orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=True, omp=True), yt)


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("add", [False, True])
@pytest.mark.parametrize("geom", GEOMS[:10], ids=str)
def test_scatter_vs_numpy_slices(geom, add, transpose):
    (H, W), bs, bst, bo, N = geom
    C = 3
    rng = np.random.default_rng(5)
    bc = bcount_covering(H, W, bst, bo)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    idx, cnt = orc.reduce_mask(mask, bc, bs, bst, bo, float(np.percentile(mask, 40)), False)
    a = active((idx, cnt))
    M = len(a)
    shape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
    blocks = rng.standard_normal(shape).astype(np.float32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    overlap = bst[0] < bs[0] or bst[1] < bs[1]
    y = orc.sparse_scatter(blocks, cnt, idx, base, bs, bst, bo, add=add, atomic=overlap, transpose=transpose)
    np.testing.assert_array_equal(y, np_scatter(blocks, a, base, bs, bst, bo, add, transpose))
    # in-place variant gives the same result and really aliases
    b2 = base.copy()
    out = orc.sparse_scatter_var(blocks, cnt, idx, b2, bs, bst, bo, add=add, atomic=overlap, transpose=transpose)
    assert out is b2
    np.testing.assert_array_equal(b2, y)


def test_scatter_roundtrip_offset_base():
    """scatter(gather(x)) over a constant base restores x where a block covers the pixel and leaves
    the base elsewhere (test_sparse_blocks.py:161, 228-239)."""
    rng = np.random.default_rng(9)
    N, H, W, C = 2, 20, 30, 5
    bs, bst, bo = (3, 4), (4, 5), (-1, -2)
    bc = bcount_covering(H, W, bst, bo)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    idx, cnt = orc.reduce_mask(mask, bc, bs, bst, bo, 0.3, False)
    g = orc.sparse_gather(x, cnt, idx, bs, bst, bo)
    y = orc.sparse_scatter(g, cnt, idx, x * 0 + 10.0, bs, bst, bo, add=False)
    covered = np.zeros((N, H, W), bool)
    for n, bh, bw in active((idx, cnt)):
        h0, w0 = bo[0] + bh * bst[0], bo[1] + bw * bst[1]
        covered[n, max(h0, 0):max(h0 + bs[0], 0), max(w0, 0):max(w0 + bs[1], 0)] = True
    np.testing.assert_array_equal(y[covered], x[covered])
    assert np.all(y[~covered] == 10.0) and covered.any() and (~covered).any()


def test_scatter_overlapping_add_vs_torch_fold():
    """All blocks active, stride < size: scatter-add is torch's fold (col2im) of the block stack."""
    rng = np.random.default_rng(13)
    N, C, H, W = 2, 4, 12, 16
    bs, bst = (4, 4), (2, 2)
    bc = [(H - bs[0]) // bst[0] + 1, (W - bs[1]) // bst[1] + 1]
    idx = np.array([(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1])], np.int16)
    M = len(idx)
    # small integers keep every partial sum exact, so fold's internal order cannot matter
    blocks = rng.integers(-8, 9, size=(M, C, bs[0], bs[1])).astype(np.float32)
    cols = torch.from_numpy(blocks).reshape(N, bc[0] * bc[1], C * bs[0] * bs[1]).permute(0, 2, 1)
    exp = F.fold(cols, (H, W), kernel_size=bs, stride=bst).permute(0, 2, 3, 1).numpy()
    y = orc.sparse_scatter(blocks, [M], idx, np.zeros((N, H, W, C), np.float32), bs, bst, [0, 0], add=True,
                           atomic=True, transpose=True)
    np.testing.assert_array_equal(y, exp)
    y2 = orc.sparse_scatter(np.ascontiguousarray(blocks.transpose(0, 2, 3, 1)), [M], idx,
                            np.zeros((N, H, W, C), np.float32), bs, bst, [0, 0], add=True, atomic=True)
    np.testing.assert_array_equal(y2, exp)


def test_scatter_add_order_is_block_major():
    """Overlapping adds accumulate in list order (sequential functor); values chosen so order shows."""
    idx = np.array([(0, 0, 0), (0, 0, 1), (0, 0, 2)], np.int16)
    blocks = np.array([1e8, 1.0, -1e8], np.float32).reshape(3, 1, 1, 1)
    y = orc.sparse_scatter(blocks, [3], idx, np.zeros((1, 1, 1, 1), np.float32), [1, 1], [1, 1], [0, 0],
                           add=True, atomic=True)
    # bstride 1 with bsize 1 puts the three blocks on different pixels; use stride 0-like overlap instead
    assert y.shape == (1, 1, 1, 1)
    base = np.zeros((1, 1, 3, 1), np.float32)
    idx2 = np.array([(0, 0, 0), (0, 0, 1)], np.int16)
    b2 = np.array([[1e8, 1.0], [-1e8, 1.0]], np.float32).reshape(2, 1, 2, 1)
    y = orc.sparse_scatter(b2, [2], idx2, base, [1, 2], [1, 1], [0, 0], add=True, atomic=True)
    # pixel 1 receives 1.0 (block 0) then -1e8 (block 1): 0 + 1.0 + -1e8
    assert y[0, 0].reshape(-1).tolist() == [1e8, np.float32(np.float32(1.0) + np.float32(-1e8)), 1.0]


def test_scatter_validation_order_and_messages():
    blocks = np.zeros((1, 2, 2, 1), np.float32)
    idx = np.zeros((1, 3), np.int16)
    base = np.zeros((1, 4, 4, 1), np.float32)
    with pytest.raises(orc.InvalidArgument, match="Only non-overlapping blocks"):
        orc.sparse_scatter(blocks, [1], idx, base, [2, 2], [1, 2], [0, 0], add=True, atomic=False)
    # overlap is fine with atomic=True or add=False (sparse_gather.cc:322-326)
    orc.sparse_scatter(blocks, [1], idx, base, [2, 2], [1, 1], [0, 0], add=True, atomic=True)
    orc.sparse_scatter(blocks, [1], idx, base, [2, 2], [1, 1], [0, 0], add=False)
    with pytest.raises(orc.InvalidArgument, match="rank 4"):
        orc.sparse_scatter(blocks, [1], idx, base[0], [2, 2], [2, 2], [0, 0], add=False)
    # the overlap rule is tested before the rank (sparse_gather.cc:322-327)
    with pytest.raises(orc.InvalidArgument, match="Only non-overlapping blocks"):
        orc.sparse_scatter(blocks, [1], idx, base[0], [2, 2], [1, 1], [0, 0], add=True, atomic=False)
    with pytest.raises(orc.InvalidArgument, match="one-dimensional"):
        orc.sparse_scatter(blocks, [1], idx, base, [2, 2, 2], [2, 2], [0, 0], add=False)
    with pytest.raises(orc.InvalidArgument, match="rank 4"):
        orc.sparse_gather(base[0], [1], idx, [2, 2], [2, 2], [0, 0])


def test_omp_rows_match_sequential():
    rng = np.random.default_rng(17)
    N, H, W, C = 2, 64, 64, 8
    bs, bst, bo = (10, 10), (8, 8), (-1, -1)
    bc = [8, 8]
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    mask = (rng.random((N, H, W, 1)) < 0.02).astype(np.float32)
    idx, cnt = orc.reduce_mask(mask, bc, bs, bst, bo, 0.5, False)
    M = int(cnt[0])
    g = orc.sparse_gather(x, cnt, idx, bs, bst, bo)
    np.testing.assert_array_equal(g, orc.sparse_gather(x, cnt, idx, bs, bst, bo, omp=True))
    y1 = orc.sparse_scatter_raw(g, M, idx, np.zeros_like(x), bs, bst, bo, add=False, transpose=False)
    y2 = orc.sparse_scatter_raw(g, M, idx, np.zeros_like(x), bs, bst, bo, add=False, transpose=False, omp=True)
    np.testing.assert_array_equal(y1, y2)
