"""Parity of the HIP kernels (through the C ABI, via sbnet_amd.ops) with the CPU oracle.

Bars: active-block lists and bin_counts bit-exact *including order* (the kernels write the CPU
functor's lexicographic order); gather and non-atomic scatter bit-exact in fp32; atomic
scatter-add on overlapping blocks within 1e-6 relative (tolerance defined in `assert_atomic_close`).

The case menu is the reference's own (sbnet_ops/tests/test_sparse_blocks.py:345-449) plus the five
benchmark configurations at full size and the hand-written vectors of tests/golden.
"""
import json
import os

import numpy as np
import pytest
import torch

import sbnet_amd
from sbnet_amd import ops, workloads
from closed_forms import box_sum_valid
from oracle import sbnet_oracle as orc

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "known_answers.json")) as f:
    GOLD = json.load(f)

DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.detach().cpu().numpy()


def bcount_covering(H, W, bstride, boffset):
    return [1 + (H - boffset[0] - 1) // bstride[0], 1 + (W - boffset[1] - 1) // bstride[1]]


def assert_atomic_close(got, exp, mag):
    """The "1e-6 relative" bar for atomic scatter-add: |got - exp| <= 1e-6 * mag element-wise, where mag is
    the same scatter-add applied to absolute values (|base| + sum of |addends| per element).  Hardware atomics
    add the few contributions of a pixel in arbitrary order; any two orders of n fp32 additions differ by at
    most 2*(n-1)*2^-24 * sum|addends| (n <= 5 here: under 5e-7 * mag), whereas an error measured against
    |exp| alone is unbounded when the addends cancel."""
    err = np.abs(got.astype(np.float64) - exp.astype(np.float64))
    bad = err > 1e-6 * mag.astype(np.float64)
    assert not bad.any(), "max err/mag %g" % float((err / np.maximum(mag, 1e-30)).max())
    # and norm-wise
    assert float(err.max()) <= 1e-6 * max(float(np.abs(exp).max()), 1e-30) * 4


def check_reduce(mask, bc, bs, bst, bo, tol, avgpool):
    """Runs reduce_mask on both sides, asserts equality and returns (host idx, host count, device idx)."""
    idx_o, cnt_o = orc.reduce_mask(mask, bc, bs, bst, bo, tol, avgpool)
    r = sbnet_amd.reduce_mask(dev(mask), bc, bs, bst, bo, tol=tol, avgpool=avgpool)
    assert r.bin_counts.dtype == torch.int32 and not r.bin_counts.is_cuda
    M = int(cnt_o[0])
    assert int(r.bin_counts[0]) == M
    assert r.active_block_indices.shape == (mask.shape[0] * bc[0] * bc[1], 3)
    np.testing.assert_array_equal(host(r.active_block_indices)[:M], idx_o[:M])
    return idx_o, cnt_o, r


def run_case(shape, RS, UV, BOFFS=(-1, -2), sparsity=70, do_add=False, N=1, test_var=False, avgpool=False,
             use_atomics=False, seed=0):
    """One runTestForOneSize of the reference's integration test, both transposes."""
    H, W, C = shape
    rng = np.random.default_rng(seed)
    bc = bcount_covering(H, W, UV, BOFFS)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    tol = float(np.percentile(x, sparsity)) if sparsity != 100 else 1e32
    idx_o, cnt_o, r = check_reduce(mask, bc, RS, UV, BOFFS, tol, avgpool)
    if sparsity == 100:
        assert int(cnt_o[0]) == 1 and idx_o[0].tolist() == [0, 0, 0]
    xd = dev(x)
    base = (x * 0.0 + 10.0).astype(np.float32)
    overlap = UV[0] < RS[0] or UV[1] < RS[1]
    g_ut = None
    for transpose in (False, True):
        g_o = orc.sparse_gather(x, cnt_o, idx_o, RS, UV, BOFFS, transpose=transpose)
        g = sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, RS, UV, BOFFS, transpose=transpose)
        assert tuple(g.shape) == g_o.shape
        np.testing.assert_array_equal(host(g), g_o)
        if not transpose:
            g_ut = g_o
        else:
            np.testing.assert_array_equal(host(g), g_ut.transpose(0, 3, 1, 2))
        if do_add and overlap and not use_atomics:
            continue
        y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, base, RS, UV, BOFFS, add=do_add, atomic=use_atomics,
                                 transpose=transpose)
        bd = dev(base)
        fn = sbnet_amd.sparse_scatter_var if test_var else sbnet_amd.sparse_scatter
        y = fn(g, r.bin_counts, r.active_block_indices, bd, RS, UV, BOFFS, add=do_add, atomic=use_atomics,
               transpose=transpose)
        if test_var:
            assert y.data_ptr() == bd.data_ptr()
        else:
            np.testing.assert_array_equal(host(bd), base)  # the copying op leaves ybase alone
        pull = not transpose and -(-RS[0] // UV[0]) <= 2 and -(-RS[1] // UV[1]) <= 2
        if do_add and use_atomics and overlap and not pull:
            mag = orc.sparse_scatter(np.abs(g_o), cnt_o, idx_o, np.abs(base), RS, UV, BOFFS, add=True, atomic=True,
                                     transpose=transpose)
            assert_atomic_close(host(y), y_o, mag)
        else:
            # add=False on overlaps writes equal values from every covering block, so order cannot matter;
            # atomic adds of an NHWC stack with at most 2x2 blocks per pixel take the atomic-free path, which
            # accumulates in the CPU functor's order and is therefore exact
            np.testing.assert_array_equal(host(y), y_o)


# ---------------------------------------------------------------------------------------------
# golden vectors
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("case", GOLD["reduce_mask"], ids=lambda c: c["name"])
def test_reduce_mask_golden(case):
    mask = np.asarray(case["mask"], np.float32)[None, :, :, None]
    r = sbnet_amd.reduce_mask(dev(mask), case["bcount"], case["bsize"], case["bstride"], case["boffset"],
                              tol=case["tol"], avgpool=case["avgpool"])
    M = int(r.bin_counts[0])
    assert host(r.active_block_indices)[:M].tolist() == case["expected_indices"]


@pytest.mark.parametrize("case", GOLD["gather_arange"], ids=lambda c: c["name"])
def test_gather_arange_golden(case):
    H, W = case["shape"]
    x = np.arange(H * W, dtype=np.float32).reshape(1, H, W, 1)
    idx = np.asarray(case["indices"], np.int16)
    y = sbnet_amd.sparse_gather(dev(x), [len(idx)], dev(idx), case["bsize"], case["bstride"], case["boffset"])
    assert host(y).reshape(len(idx), -1).tolist() == case["expected_blocks"]


@pytest.mark.parametrize("use_var", [False, True])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("case", GOLD["pipeline"], ids=lambda c: c["name"])
def test_pipeline_known_answers(case, transpose, use_var):
    mask = np.asarray(case["mask"], np.float32)[None, :, :, None]
    x = np.ones_like(mask)
    r = sbnet_amd.reduce_mask(dev(mask), case["bcount"], case["bsize"], case["bstride"], case["boffset"], tol=0.0)
    p = sbnet_amd.sparse_gather(dev(x), r.bin_counts, r.active_block_indices, case["bsize"], case["bstride"],
                                case["boffset"], transpose=transpose)
    p = host(p)
    q = box_sum_valid(p.transpose(0, 2, 3, 1) if transpose else p, case["ksize"][0], case["ksize"][1],
                      *case["conv_strides"])
    if transpose:
        q = np.ascontiguousarray(q.transpose(0, 3, 1, 2))
    y_exp = np.asarray(case["y_exp"], np.float32)[None, :, :, None]
    fn = sbnet_amd.sparse_scatter_var if use_var else sbnet_amd.sparse_scatter
    y = fn(dev(q), r.bin_counts, r.active_block_indices, dev(np.zeros_like(y_exp)), case["bsize_out"],
           case.get("s_bstride", case["bstride"]), [0, 0], add=False, transpose=transpose)
    np.testing.assert_array_equal(host(y), y_exp)


# ---------------------------------------------------------------------------------------------
# the reference integration test's case list
# ---------------------------------------------------------------------------------------------

def test_simple():
    run_case((2, 3, 2), RS=(2, 3), UV=(3, 4))
    run_case((5, 5, 1), RS=(3, 3), UV=(1, 1))


def test_zero_block_count():
    run_case((2, 2, 1), RS=(1, 1), UV=(1, 1), BOFFS=(0, 0), sparsity=100)
    run_case((40, 40, 8), RS=(5, 5), UV=(5, 5), BOFFS=(0, 0), sparsity=100, avgpool=True, N=3)


def test_basic_and_overlapping():
    run_case((2, 2, 1), RS=(1, 1), UV=(1, 1), BOFFS=(0, 0), sparsity=0)
    run_case((2, 2, 1), RS=(1, 1), UV=(1, 1), BOFFS=(0, 0), sparsity=0, N=3)
    run_case((6, 6, 1), RS=(1, 1), UV=(1, 1))
    run_case((3, 3, 1), RS=(2, 2), UV=(1, 1), BOFFS=(0, 0), sparsity=0)
    run_case((13, 12, 1), RS=(2, 3), UV=(1, 2), BOFFS=(0, 0), sparsity=0.1)


@pytest.mark.parametrize("sparsity", [10, 20, 30, 40, 50, 70, 90, 99])
def test_sparsities(sparsity):
    # avg pooling over a Gaussian (non-binary) mask: decisions must follow the CPU summation order
    run_case((200, 300, 32), RS=(3, 4), UV=(2, 3), sparsity=sparsity, avgpool=True, use_atomics=True)


def test_avg_pooling_with_holes():
    run_case((2, 3, 2), RS=(2, 3), UV=(3, 4), avgpool=True)
    run_case((2, 3, 2), RS=(2, 3), UV=(3, 4), avgpool=False)


@pytest.mark.parametrize("cc", [15, 16, 24, 32, 48, 64])
def test_channel_sweep(cc):
    run_case((380, 480, cc), RS=(18, 18), UV=(18, 18))


def test_channel_sweep_16():
    run_case((200, 300, 32), RS=(16, 16), UV=(16, 16))


@pytest.mark.parametrize("avgpool", [True, False])
@pytest.mark.parametrize("tv", [True, False])
@pytest.mark.parametrize("nn", [1, 7])
def test_simple_permutations(nn, tv, avgpool):
    for sp in [0, 10, 50, 99]:
        args = dict(RS=(1, 1), UV=(1, 1), BOFFS=[0, 0], sparsity=sp, N=nn, test_var=tv, avgpool=avgpool)
        for shape in [(1, 1, 1), (1, 1, 2), (1, 2, 3), (2, 1, 3), (3, 2, 1), (1, 2, 1), (3, 2, 7)]:
            run_case(shape, **args)
    run_case((1, 1, 1024 * 49), RS=(1, 1), UV=(1, 1), BOFFS=[0, 0], sparsity=50, N=nn, test_var=tv,
             avgpool=avgpool)


def test_uneven_gaps_offsets():
    run_case((8, 10, 7), RS=(3, 4), UV=(3, 4))
    run_case((8, 10, 1), RS=(3, 4), UV=(4, 5))
    run_case((8, 10, 7), RS=(3, 4), UV=(4, 5))
    run_case((5, 5, 1), RS=(3, 2), UV=(3, 2), BOFFS=[-1, -2])
    run_case((5, 3, 1), RS=(2, 3), UV=(2, 3), BOFFS=[0, 0])
    run_case((5, 3, 1), RS=(2, 3), UV=(2, 3), BOFFS=[-1, -2])
    run_case((3, 3, 1), RS=(2, 2), UV=(1, 1), BOFFS=[0, 0])
    run_case((3, 3, 1), RS=(1, 1), UV=(2, 2))


def test_large_block_sizes():
    run_case((2048, 2048, 1), RS=(1500, 490), UV=(300, 390), use_atomics=True)


@pytest.mark.parametrize("C", [1, 2, 3, 6, 7, 12, 20, 128, 130])
@pytest.mark.parametrize("do_add", [False, True])
def test_odd_channels_and_adds(C, do_add):
    run_case((33, 47, C), RS=(5, 7), UV=(5, 7), BOFFS=(-2, -3), sparsity=40, do_add=do_add, N=2, seed=C)
    run_case((33, 47, C), RS=(5, 7), UV=(3, 4), BOFFS=(-2, -3), sparsity=40, do_add=do_add, N=2,
             use_atomics=True, seed=C + 100)


def test_misaligned_base_pointers():
    """Tensors whose storage starts 4 or 8 bytes past a 16-byte boundary take the narrower vector paths."""
    rng = np.random.default_rng(21)
    N, H, W, C = 2, 20, 24, 8
    bs, bst, bo = (5, 6), (5, 6), (-1, -1)
    bc = bcount_covering(H, W, bst, bo)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    idx_o, cnt_o, r = check_reduce(mask, bc, bs, bst, bo, 0.2, False)
    for off in (1, 2, 3):
        buf = torch.zeros(x.size + 8, dtype=torch.float32, device=DEV)
        xd = buf[off:off + x.size].view(N, H, W, C)
        xd.copy_(torch.from_numpy(x))
        assert xd.data_ptr() % 16 == 4 * off
        for transpose in (False, True):
            g_o = orc.sparse_gather(x, cnt_o, idx_o, bs, bst, bo, transpose=transpose)
            gbuf = torch.zeros(g_o.size + 8, dtype=torch.float32, device=DEV)
            gout = gbuf[off:off + g_o.size].view(*g_o.shape)
            sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, bs, bst, bo, transpose=transpose,
                                    out=gout)
            np.testing.assert_array_equal(host(gout), g_o)
            ybuf = torch.full((x.size + 8,), 10.0, dtype=torch.float32, device=DEV)
            yd = ybuf[off:off + x.size].view(N, H, W, C)
            sbnet_amd.sparse_scatter_var(gout, r.bin_counts, r.active_block_indices, yd, bs, bst, bo, add=True,
                                         transpose=transpose)
            y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, np.full_like(x, 10.0), bs, bst, bo, add=True,
                                     transpose=transpose)
            np.testing.assert_array_equal(host(yd), y_o)
            assert float(ybuf[:off].min()) == 10.0 and float(ybuf[off + x.size:].max()) == 10.0


@pytest.mark.parametrize("geom", [
    # (H, W, C), bsize, bstride, boffset, out offset in floats, N
    ((120, 130, 128), (27, 27), (25, 25), (-1, -1), 0, 1),    # 3 splits per plane, chunks start on 128-byte lines
    ((120, 130, 128), (27, 27), (25, 25), (-1, -1), 4, 1),    # same, output 16 bytes past a line
    ((120, 130, 128), (27, 27), (25, 25), (-1, -1), 20, 2),   # 80 bytes past a line
    ((120, 130, 20), (27, 27), (25, 25), (-1, -1), 0, 1),     # one partial chunk (20 of 32 channels), odd chunk starts
    ((120, 130, 48), (27, 27), (25, 25), (-1, -1), 8, 2),     # full chunk + partial chunk
    ((100, 90, 16), (21, 23), (20, 20), (-3, -2), 0, 1),      # 483-pixel planes, 2 splits, 16-channel chunks
    ((100, 90, 36), (19, 17), (19, 17), (0, 0), 12, 1),       # 323-pixel planes
    ((64, 64, 8), (5, 5), (5, 5), (0, 0), 0, 3),              # planes shorter than a line: a line crosses two planes
    ((64, 64, 8), (5, 5), (5, 5), (0, 0), 28, 3),
    ((64, 64, 32), (3, 3), (2, 2), (-1, -1), 0, 1),           # 9-pixel planes
    ((64, 64, 4), (9, 7), (9, 7), (0, 0), 4, 2),              # single 4-channel vector per pixel
    ((300, 300, 32), (32, 32), (32, 32), (0, 0), 0, 1),       # planes that are whole lines, 5 splits
    ((300, 300, 32), (33, 31), (30, 30), (-2, -2), 16, 1),
])
def test_planar_gather_owns_whole_lines(geom):
    """Planar gather into outputs at every kind of alignment against 128-byte lines: the kernel assigns whole
    lines of the stack to workgroups, so chunk starts, split points and plane ends that fall inside a line are
    the cases to cover; guard zones around the output must stay untouched."""
    (H, W, C), bs, bst, bo, off, N = geom
    rng = np.random.default_rng(H * 7 + C + off)
    bc = bcount_covering(H, W, bst, bo)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    cells = rng.random((N, bc[0], bc[1])) < 0.6
    cells[0, 0, 0] = cells[-1, -1, -1] = True
    idx = np.ascontiguousarray(np.argwhere(cells), dtype=np.int16)
    rng.shuffle(idx, axis=0)  # the op takes any list order
    cnt = np.array([idx.shape[0]], dtype=np.int32)
    g_o = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=True)
    guard = 64
    gbuf = torch.full((g_o.size + off + 2 * guard,), 777.0, dtype=torch.float32, device=DEV)
    assert gbuf.data_ptr() % 128 == 0
    gout = gbuf[guard + off:guard + off + g_o.size].view(*g_o.shape)
    sbnet_amd.sparse_gather(dev(x), cnt, dev(idx), bs, bst, bo, transpose=True, out=gout)
    np.testing.assert_array_equal(host(gout), g_o)
    assert float(gbuf[:guard + off].min()) == 777.0 and float(gbuf[:guard + off].max()) == 777.0
    assert float(gbuf[guard + off + g_o.size:].min()) == 777.0 and float(gbuf[guard + off + g_o.size:].max()) == 777.0
    # and back: the planar scatter restores exactly the gathered pixels
    yd = torch.zeros((N, H, W, C), dtype=torch.float32, device=DEV)
    sbnet_amd.sparse_scatter_var(gout, cnt, dev(idx), yd, bs, bst, bo, add=False, transpose=True)
    y_o = orc.sparse_scatter(g_o, cnt, idx, np.zeros_like(x), bs, bst, bo, add=False, transpose=True)
    np.testing.assert_array_equal(host(yd), y_o)


# ---------------------------------------------------------------------------------------------
# reduce_mask: summation order, thresholds, sizes
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("bs,bst", [((6, 6), (4, 4)), ((18, 18), (16, 16)), ((27, 27), (25, 25)), ((3, 50), (3, 45)),
                                    ((64, 2), (60, 2)), ((40, 40), (10, 10))])
def test_reduce_mask_avg_order_sensitive(bs, bst):
    """Masks built so that fp32 summation order changes block sums, with thresholds sitting on the
    sequential sums themselves: any deviation from the row-major order flips decisions."""
    rng = np.random.default_rng(bs[0] * 100 + bs[1])
    N, H, W = 3, 160, 190
    bo = (-1, -1)
    bc = bcount_covering(H, W, bst, bo)
    mask = (rng.standard_normal((N, H, W, 1)) * rng.choice([1e-3, 1.0, 1e4], size=(N, H, W, 1))).astype(np.float32)
    # thresholds: the exact sequential average of a few blocks (ties) and values one ulp either side
    sums = []
    for n, bh, bw in [(0, 1, 1), (1, 2, 3), (2, 0, 0), (1, bc[0] - 1, bc[1] - 1)]:
        h0, w0 = bo[0] + bh * bst[0], bo[1] + bw * bst[1]
        s = np.float32(0)
        for hh in range(max(h0, 0), min(h0 + bs[0], H)):
            for ww in range(max(w0, 0), min(w0 + bs[1], W)):
                s = np.float32(s + mask[n, hh, ww, 0])
        sums.append(np.float32(s / np.float32(bs[0] * bs[1])))
    for t in sums:
        for tol in (t, np.nextafter(t, np.float32(-np.inf)), np.nextafter(t, np.float32(np.inf))):
            check_reduce(mask, bc, bs, bst, bo, float(tol), True)
    check_reduce(mask, bc, bs, bst, bo, 0.0, True)


def test_reduce_mask_special_values():
    rng = np.random.default_rng(5)
    N, H, W = 2, 64, 64
    bs, bst, bo = (9, 9), (8, 8), (-1, -1)
    bc = [8, 8]
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    mask[0, 3, 3, 0] = np.inf
    mask[0, 20, 20, 0] = -np.inf
    mask[0, 40, 40, 0] = np.nan
    mask[1, 10, 10, 0] = np.inf
    mask[1, 11, 11, 0] = -np.inf
    mask[1, 50, 50, 0] = 3e38
    mask[1, 51, 51, 0] = 3e38
    for avg in (False, True):
        for tol in (-1.0, 0.0, 0.05, 1e30):
            check_reduce(mask, bc, bs, bst, bo, tol, avg)


def test_reduce_mask_many_blocks_and_async_count():
    rng = np.random.default_rng(8)
    N, H, W = 5, 300, 300
    mask = (rng.random((N, H, W, 1)) < 0.3).astype(np.float32)
    bc = bcount_covering(H, W, (2, 2), (0, 0))
    idx_o, cnt_o, r = check_reduce(mask, bc, (2, 2), (2, 2), (0, 0), 0.4, True)
    r2 = sbnet_amd.reduce_mask(dev(mask), bc, (2, 2), (2, 2), (0, 0), tol=0.4, avgpool=True, sync=False)
    assert r2.bin_counts.is_cuda
    torch.cuda.synchronize()
    assert int(r2.bin_counts[0]) == int(cnt_o[0])
    np.testing.assert_array_equal(host(r2.active_block_indices)[:int(cnt_o[0])], idx_o[:int(cnt_o[0])])


def test_reduce_mask_four_million_blocks():
    """N = 64 images of 256x256 one-pixel blocks: 4 194 304 blocks, 16 384 pooling workgroups whose counts go
    through the prefix-sum kernel.  Order and count against the oracle, and the three launches take far less than
    the time a compaction that re-sums all earlier counts in every workgroup would."""
    rng = np.random.default_rng(77)
    N, H, W = 64, 256, 256
    mask = (rng.random((N, H, W, 1)) < 0.3).astype(np.float32)
    bc, bs, bst, bo = [H, W], [1, 1], [1, 1], [0, 0]
    idx_o, cnt_o = orc.reduce_mask(mask, bc, bs, bst, bo, 0.5, False)
    M = int(cnt_o[0])
    md = dev(mask)
    r = sbnet_amd.reduce_mask(md, bc, bs, bst, bo, tol=0.5, avgpool=False)
    assert int(r.bin_counts[0]) == M
    assert torch.equal(r.active_block_indices[:M].cpu(), torch.from_numpy(idx_o[:M]))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        sbnet_amd.reduce_mask(md, bc, bs, bst, bo, tol=0.5, avgpool=False, sync=False)
    e1.record()
    e1.synchronize()
    assert e0.elapsed_time(e1) / 5 < 5.0, "reduce_mask over 4M blocks took %.2f ms" % (e0.elapsed_time(e1) / 5)


@pytest.mark.parametrize("bs,bst,bo", [((2, 2), (2, 2), (0, 0)), ((3, 3), (2, 2), (-1, -1))])
def test_more_blocks_than_a_launch_dimension_holds(bs, bst, bo):
    """More than 65 535 active blocks: the planar kernels then number their workgroups along one launch
    dimension instead of (tiles, blocks).  Whole pipeline, both stack layouts."""
    rng = np.random.default_rng(21)
    N, H, W, C = 1200, 16, 16, 8
    mask = (rng.random((N, H, W, 1)) < 0.97).astype(np.float32)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    bc = [8, 8]
    idx_o, cnt_o, r = check_reduce(mask, bc, bs, bst, bo, 0.5, False)
    assert int(cnt_o[0]) > 65535
    xd = dev(x)
    for transpose in (False, True):
        g_o = orc.sparse_gather(x, cnt_o, idx_o, bs, bst, bo, transpose=transpose)
        g = sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, bs, bst, bo, transpose=transpose)
        np.testing.assert_array_equal(host(g), g_o)
        base = np.full_like(x, 3.0)
        y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, base, bs, bst, bo, add=False, transpose=transpose)
        y = sbnet_amd.sparse_scatter_var(g, r.bin_counts, r.active_block_indices, dev(base), bs, bst, bo, add=False,
                                         transpose=transpose)
        np.testing.assert_array_equal(host(y), y_o)


def test_image_of_2_pow_30_floats_takes_the_64_bit_offset_kernels():
    """An image of 2^30 floats (4 GiB) is the first size whose byte offsets do not fit 32 bits: gather and
    scatter then leave the buffer-addressed kernels for the ones with 64-bit addressing (NHWC stack) and the
    one-thread-per-element kernel (planar stack).  Blocks at the far end of the image, where offsets exceed
    2^32, against the oracle; in-place scatter checked on the whole 4 GiB tensor."""
    N, H, W, C = 1, 8192, 8192, 16
    bs, bst, bo = (5, 6), (6, 7), (-1, -2)
    g = torch.Generator(device=DEV).manual_seed(5)
    xd = torch.randint(-1000, 1000, (N, H, W, C), generator=g, device=DEV, dtype=torch.int32).to(torch.float32)
    x = host(xd)
    bh_max, bw_max = (H - bo[0] - 1) // bst[0], (W - bo[1] - 1) // bst[1]
    idx = np.array([[0, 0, 0], [0, bh_max, bw_max], [0, bh_max, 0], [0, bh_max - 1, bw_max - 3], [0, 1500, 77],
                    [0, bh_max // 2 + 1, bw_max], [0, 0, bw_max]], np.int16)
    cnt = np.array([len(idx)], np.int32)
    idx_d, cnt_t = dev(idx), torch.from_numpy(cnt)
    for transpose in (False, True):
        g_o = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=transpose)
        gd = sbnet_amd.sparse_gather(xd, cnt_t, idx_d, bs, bst, bo, transpose=transpose)
        np.testing.assert_array_equal(host(gd), g_o)
        stack = (g_o * 0.5 + 1.0).astype(np.float32)
        y_o = orc.sparse_scatter_var(stack, cnt, idx, x.copy(), bs, bst, bo, add=True, transpose=transpose)
        yd = xd.clone()
        sbnet_amd.sparse_scatter_var(dev(stack), cnt_t, idx_d, yd, bs, bst, bo, add=True, transpose=transpose)
        assert torch.equal(yd, dev(y_o))
        del yd, y_o
    del xd, x
    torch.cuda.empty_cache()


def test_host_visible_count_is_never_stale_and_threads_do_not_mix():
    """The host-visible count arrives through a polled word of pinned memory, one per thread: many calls in a row
    with alternating masks must each report their own count, and two threads on two streams must not see each
    other's; a call under stream capture must fail instead of waiting for a kernel that does not run."""
    import threading
    rng = np.random.default_rng(77)
    H, W = 96, 96
    bs, bst, bo = (8, 8), (8, 8), (0, 0)
    bc = [12, 12]
    masks = [(rng.random((1, H, W, 1)) < p).astype(np.float32) for p in (0.0005, 0.002, 0.01, 0.0)]
    want = [int(orc.reduce_mask(m, bc, bs, bst, bo, 0.5, False)[1][0]) for m in masks]
    assert len(set(want)) == len(want)
    md = [dev(m) for m in masks]
    for i in range(200):
        r = sbnet_amd.reduce_mask(md[i % 4], bc, bs, bst, bo, tol=0.5)
        assert int(r.bin_counts[0]) == want[i % 4]

    errors = []

    def worker(first):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for i in range(150):
                    k = (first + i) % 4
                    r = sbnet_amd.reduce_mask(md[k], bc, bs, bst, bo, tol=0.5)
                    if int(r.bin_counts[0]) != want[k]:
                        errors.append((first, i, int(r.bin_counts[0]), want[k]))
                        return
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(f,)) for f in (0, 1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sbnet_amd.reduce_mask(md[0], bc, bs, bst, bo, tol=0.5, sync=False)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    failed = False
    with torch.cuda.graph(graph):
        try:
            sbnet_amd.reduce_mask(md[0], bc, bs, bst, bo, tol=0.5)  # host count: not possible while capturing
        except RuntimeError:
            failed = True
        sbnet_amd.reduce_mask(md[0], bc, bs, bst, bo, tol=0.5, sync=False)
    assert failed
    torch.cuda.synchronize()


@pytest.mark.parametrize("geom", [
    # (N, H, W, C), bsize, bstride, boffset, keep probability, add
    ((2, 200, 200, 64), (16, 16), (16, 16), (0, 0), 0.9, True),
    ((2, 200, 200, 64), (16, 16), (16, 16), (0, 0), 0.9, False),
    ((2, 256, 256, 64), (18, 18), (16, 16), (-1, -1), 0.8, False),   # overlapping blocks
    ((4, 256, 256, 64), (5, 7), (8, 9), (2, -3), 1.0, True),         # gaps, uneven offsets
    ((1, 512, 512, 30), (9, 9), (9, 9), (-4, 3), 0.95, True),        # 8-byte vectors
    ((1, 1200, 1100, 7), (11, 13), (11, 13), (0, 0), 1.0, True),     # 4-byte vectors
    ((1, 800, 800, 32), (27, 27), (25, 25), (-1, -1), 0.9, False),   # plane split over several tiles
    ((1, 300, 480, 64), (18, 18), (18, 18), (-1, -2), 0.5, True),    # planar stack: one launch over the cells,
    ((1, 300, 480, 64), (18, 18), (18, 18), (-1, -2), 0.5, False),   # half of them empty
    ((2, 150, 130, 256), (18, 18), (18, 18), (-1, -2), 0.3, False),  # several channel chunks
    ((1, 4500, 4000, 4), (16, 17), (16, 17), (-7, -11), 0.7, True),  # more cells than a launch has rows
], ids=lambda g: "x".join(map(str, g[0])) + "_b%dx%d_%s" % (g[1] + ("add" if g[5] else "assign",)))
def test_copying_scatter_moves_every_byte_once(geom):
    """sparse_scatter (the op that returns a new tensor) with enough coverage builds its output from two disjoint
    parts -- pixels no active block covers are copied from ybase, covered ones written by the scatter, which
    reads ybase where it adds -- instead of copying ybase and scattering on top.  Same result, bit for bit, for
    both stack layouts, with the count on the host and on the device; ybase is left alone."""
    (N, H, W, C), bs, bst, bo, keep, add = geom
    rng = np.random.default_rng(hash(geom[0]) % 1000)
    bc = bcount_covering(H, W, bst, bo)
    allb = np.array([(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1])], np.int16)
    idx = allb[rng.random(len(allb)) < keep]
    cnt = np.array([len(idx)], np.int32)
    # enough coverage for the one-pass path (the launch over cells of blocks that tile the plane needs none)
    assert len(idx) * bs[0] * bs[1] * C * 4 >= 16 << 20 or tuple(bs) == tuple(bst)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    idx_d, cnt_t, base_d = dev(idx), torch.from_numpy(cnt), dev(base)
    cnt_d = cnt_t.to(DEV)
    for transpose in (False, True):
        stack = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=transpose)   # overlaps carry equal values
        y_o = orc.sparse_scatter(stack, cnt, idx, base, bs, bst, bo, add=add, transpose=transpose)
        stack_d = dev(stack)
        y = sbnet_amd.sparse_scatter(stack_d, cnt_t, idx_d, base_d, bs, bst, bo, add=add, transpose=transpose)
        assert y.data_ptr() != base_d.data_ptr()
        np.testing.assert_array_equal(host(y), y_o)
        y2 = sbnet_amd.sparse_scatter(stack_d, cnt_d, idx_d, base_d, bs, bst, bo, add=add, transpose=transpose)
        np.testing.assert_array_equal(host(y2), y_o)
        np.testing.assert_array_equal(host(base_d), base)
    # a base that is only 4-byte aligned takes the narrow copies
    flat = torch.empty(base_d.numel() + 1, device=DEV)
    mis = flat[1:].view(base_d.shape)
    mis.copy_(base_d)
    y_o = orc.sparse_scatter(stack, cnt, idx, base, bs, bst, bo, add=add, transpose=True)
    y3 = sbnet_amd.sparse_scatter(stack_d, cnt_t, idx_d, mis, bs, bst, bo, add=add, transpose=True)
    np.testing.assert_array_equal(host(y3), y_o)


@pytest.mark.parametrize("geom", [
    # (N, H, W, C), bsize, bstride, boffset
    ((2, 40, 56, 32), (4, 4), (4, 4), (0, 0)),      # whole 4x4 planes: the planar stack is staged through LDS
    ((1, 64, 64, 64), (8, 8), (8, 8), (-3, 0)),     # two channel chunks, rows offset
    ((2, 30, 44, 16), (3, 4), (5, 8), (1, 0)),      # gaps between the blocks
    ((1, 33, 47, 5), (5, 7), (6, 7), (-2, -3)),     # scalar channel vectors, nothing aligned
    ((1, 70, 90, 48), (9, 10), (9, 10), (-2, -3)),  # planar stack by cells: blocks that tile the plane, odd offset
    ((2, 50, 41, 6), (13, 15), (13, 15), (0, -1)),  # the same with 8-byte channel vectors
])
def test_copying_scatter_of_a_list_with_repeated_rows(geom):
    """Non-overlapping blocks, a list that names some blocks twice or three times with different stack rows: the
    sequential CPU functor lets the last row win a plain write and adds every row, in list order, for add=True
    (sparse_gather.cc:105-129).  The copying op (built in one pass over the output) does the same, bit for bit."""
    (N, H, W, C), bs, bst, bo = geom
    rng = np.random.default_rng(H + W + C)
    bc = bcount_covering(H, W, bst, bo)
    cells = [(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1]) if rng.random() < 0.6]
    idx = np.array(cells + cells[:5] + cells[2:4], np.int16)
    rng.shuffle(idx, axis=0)
    M = len(idx)
    cnt = np.array([M], np.int32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    # planar stacks are exact for such lists where the strips stage them or the launch runs over the cells
    aligned = bs[1] % 4 == 0 and bst[1] % 4 == 0 and bo[1] % bst[1] == 0
    by_cells = tuple(bs) == tuple(bst) and bst[0] * bst[1] * C * 4 >= 4096
    for transpose in ((False, True) if aligned or by_cells else (False,)):
        shape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
        stack = (rng.standard_normal(shape) * rng.choice([1e-3, 1.0, 1e4], size=(M, 1, 1, 1))).astype(np.float32)
        for add in (False, True):
            y_o = orc.sparse_scatter(stack, cnt, idx, base, bs, bst, bo, add=add, transpose=transpose)
            y = sbnet_amd.sparse_scatter(dev(stack), cnt, dev(idx), dev(base), bs, bst, bo, add=add, transpose=transpose)
            np.testing.assert_array_equal(host(y), y_o, err_msg="transpose %s add %s" % (transpose, add))
            dcount = torch.tensor([M - 3], dtype=torch.int32, device=DEV)
            y_o2 = orc.sparse_scatter(stack, [M - 3], idx, base, bs, bst, bo, add=add, transpose=transpose)
            y = sbnet_amd.sparse_scatter(dev(stack), dcount, dev(idx), dev(base), bs, bst, bo, add=add, transpose=transpose)
            np.testing.assert_array_equal(host(y), y_o2, err_msg="device count, transpose %s add %s" % (transpose, add))


@pytest.mark.parametrize("case", [
    # (H, W, C), bsize, bstride, boffset, block list (n, bh, bw)
    ((20, 30, 8), (6, 7), (6, 7), (0, 0), []),                                   # empty list
    ((20, 30, 8), (6, 7), (6, 7), (0, 0), [(0, 50, 0), (0, 0, 90), (0, -9, -9)]),  # blocks wholly outside the image
    ((20, 30, 8), (6, 7), (6, 7), (-40, -40), [(0, 0, 0), (0, 6, 5), (0, 7, 6)]),  # far negative offsets
    ((5, 4, 12), (9, 11), (9, 11), (-2, -3), [(0, 0, 0)]),                       # a block larger than the image
    ((1, 37, 4), (1, 5), (1, 5), (0, -1), [(0, 0, 0), (0, 0, 3), (0, 0, 7)]),      # one-row image
    ((41, 1, 6), (4, 1), (4, 1), (-1, 0), [(0, 0, 0), (0, 5, 0), (0, 10, 0)]),     # one-column image
    ((16, 16, 3), (4, 4), (4, 4), (0, 0), [(1, 3, 3), (0, 0, 0), (1, 0, 0), (0, 3, 3)]),  # list not in order, N = 2
], ids=["empty", "outside", "far_offset", "block_gt_image", "one_row", "one_column", "unordered"])
def test_edge_geometries(case):
    """Lists and geometries at the edges of what the ops accept: nothing to do, blocks that miss the image
    (gather pads with zeros, scatter drops), blocks larger than the image, degenerate images, an arbitrary
    block order.  Gather and both scatters against the oracle, both stack layouts."""
    (H, W, C), bs, bst, bo, blocks = case
    N = 2
    rng = np.random.default_rng(len(blocks) + H)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    idx = np.asarray(blocks, np.int16).reshape(-1, 3)
    cnt = np.array([len(idx)], np.int32)
    idx_d = dev(idx) if len(idx) else torch.zeros((1, 3), dtype=torch.int16, device=DEV)
    idx_o = idx if len(idx) else np.zeros((1, 3), np.int16)
    cnt_t = torch.from_numpy(cnt)
    for transpose in (False, True):
        g_o = orc.sparse_gather(x, cnt, idx_o, bs, bst, bo, transpose=transpose)
        g = sbnet_amd.sparse_gather(dev(x), cnt_t, idx_d, bs, bst, bo, transpose=transpose)
        assert tuple(g.shape) == g_o.shape
        np.testing.assert_array_equal(host(g), g_o)
        stack = rng.standard_normal(g_o.shape).astype(np.float32)
        for add in (False, True):
            y_o = orc.sparse_scatter(stack, cnt, idx_o, base, bs, bst, bo, add=add, transpose=transpose)
            y = sbnet_amd.sparse_scatter(dev(stack), cnt_t, idx_d, dev(base), bs, bst, bo, add=add,
                                         transpose=transpose)
            np.testing.assert_array_equal(host(y), y_o)
            bd = dev(base)
            sbnet_amd.sparse_scatter_var(dev(stack), cnt_t, idx_d, bd, bs, bst, bo, add=add, transpose=transpose)
            np.testing.assert_array_equal(host(bd), y_o)


def test_reduce_mask_random_sweep():
    """Seeded random reduce_mask problems: image and block sizes from 1 to ~90 / ~40, strides smaller and larger than
    the blocks, offsets on either side of zero, block counts that under- and over-cover the image, binary, Gaussian
    and wide-dynamic-range masks, both pooling modes, thresholds on either side of the data.  Count and ordered list
    against the oracle."""
    for seed in range(150):
        rng = np.random.default_rng(10_000 + seed)
        N, H, W = int(rng.integers(1, 5)), int(rng.integers(1, 90)), int(rng.integers(1, 90))
        bs = (int(rng.integers(1, 40)), int(rng.integers(1, 40)))
        bst = (int(rng.integers(1, 40)), int(rng.integers(1, 40)))
        bo = (int(rng.integers(-20, 5)), int(rng.integers(-20, 5)))
        bc = [int(rng.integers(1, 12)), int(rng.integers(1, 12))]
        avg = bool(rng.integers(0, 2))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            mask = (rng.random((N, H, W, 1)) < rng.random() * 0.2).astype(np.float32)
        elif kind == 1:
            mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
        else:
            mask = (rng.standard_normal((N, H, W, 1)) * 10.0 ** rng.integers(-3, 4, (N, H, W, 1))).astype(np.float32)
        tol = float(rng.choice([0.0, 0.05, 0.5, -0.1, float(np.percentile(mask, 90))]))
        idx_o, cnt_o = orc.reduce_mask(mask, bc, bs, bst, bo, tol, avg)
        r = sbnet_amd.reduce_mask(dev(mask), bc, bs, bst, bo, tol=tol, avgpool=avg)
        M = int(cnt_o[0])
        assert int(r.bin_counts[0]) == M, (seed, N, H, W, bs, bst, bo, bc, avg, kind, tol)
        np.testing.assert_array_equal(host(r.active_block_indices)[:M], idx_o[:M], err_msg=str(seed))


def test_reduce_mask_rows_past_count_untouched():
    mask = np.zeros((1, 8, 8, 1), np.float32)
    mask[0, 0, 0, 0] = 1.0
    lib_idx = torch.full((16, 3), 77, dtype=torch.int16, device=DEV)
    # call through the raw ABI with a caller-owned index buffer
    import ctypes
    from sbnet_amd import _lib
    L = _lib.load()
    I2 = ctypes.c_int32 * 2
    nws = L.sbnet_reduce_mask_workspace_bytes(1, I2(4, 4), 2)
    ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
    cnt = np.zeros(1, np.int32)
    rc = L.sbnet_reduce_mask(dev(mask).data_ptr(), 1, 8, 8, I2(4, 4), 2, I2(2, 2), 2, I2(2, 2), 2, I2(0, 0), 2, 0.5,
                             0, lib_idx.data_ptr(), cnt.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), None,
                             ws.data_ptr(), nws, None)
    assert rc == 0 and cnt[0] == 1
    out = host(lib_idx)
    assert out[0].tolist() == [0, 0, 0] and (out[1:] == 77).all()
    # without a workspace the library allocates its own
    rc = L.sbnet_reduce_mask(dev(mask).data_ptr(), 1, 8, 8, I2(4, 4), 2, I2(2, 2), 2, I2(2, 2), 2, I2(0, 0), 2, 0.5,
                             0, lib_idx.data_ptr(), cnt.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), None,
                             None, 0, None)
    assert rc == 0 and cnt[0] == 1
    # functor level: raw count, zero stays zero and nothing is written
    lib_idx.fill_(55)
    dcnt = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    rc = L.sbnet_reduce_mask_functor(dev(mask * 0).data_ptr(), 1, 8, 8, 0.5, 0, 0, 2, 2, 2, 2, 4, 4, 1, 16,
                                     lib_idx.data_ptr(), dcnt.data_ptr(), 0, ws.data_ptr(), nws, None)
    torch.cuda.synchronize()
    assert rc == 0 and int(dcnt[0]) == 0 and (host(lib_idx) == 55).all()


# ---------------------------------------------------------------------------------------------
# overlapping scatter-add: the atomic-free path and its fall-backs
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("geom", [((40, 52, 8), (6, 6), (3, 3), (-2, -1)), ((33, 47, 5), (5, 7), (3, 4), (-2, -3)),
                                   ((64, 64, 16), (16, 16), (8, 8), (0, 0)), ((30, 30, 4), (4, 9), (4, 5), (1, 2)),
                                   ((25, 25, 12), (7, 3), (5, 3), (-6, 0))], ids=str)
def test_overlapping_add_is_exact_and_ordered(geom):
    """Values spanning many magnitudes make fp32 sums order dependent: only the CPU functor's ascending
    block order reproduces the oracle bit for bit.  The block list is shuffled, so "ascending" means list
    position, not block coordinates."""
    (H, W, C), bs, bst, bo = geom
    rng = np.random.default_rng(H * W + C)
    N = 2
    bc = bcount_covering(H, W, bst, bo)
    allb = np.array([(n, i, j) for n in range(N) for i in range(-1, bc[0] + 1) for j in range(-1, bc[1] + 1)], np.int16)
    pick = rng.random(len(allb)) < 0.6
    idx = allb[pick][rng.permutation(int(pick.sum()))]
    M = len(idx)
    stack = (rng.standard_normal((M, bs[0], bs[1], C)) * rng.choice([1e-4, 1.0, 1e5], size=(M, 1, 1, 1))).astype(np.float32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True)
    y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=True, atomic=True)
    np.testing.assert_array_equal(host(y), y_o)
    bd = dev(base)
    sbnet_amd.sparse_scatter_var(dev(stack), [M], dev(idx), bd, bs, bst, bo, add=True, atomic=True)
    np.testing.assert_array_equal(host(bd), y_o)


@pytest.mark.parametrize("geom", [
    # (N, H, W, C), bsize, bstride, boffset
    ((2, 40, 52, 8), (6, 6), (3, 3), (-2, -1)),          # 2x2 blocks per pixel
    ((1, 33, 47, 5), (5, 7), (3, 4), (-2, -3)),          # scalar channel vectors
    ((1, 30, 30, 6), (7, 7), (2, 2), (0, 0)),            # 4x4 blocks per pixel
    ((1, 64, 64, 16), (10, 10), (8, 8), (-1, -1)),       # the plumbing configuration's geometry
    ((1, 120, 130, 32), (27, 27), (25, 25), (-1, -1)),   # planes split over tiles
    ((2, 64, 72, 256), (16, 16), (8, 8), (0, 0)),        # the atomic scatter-add configuration's geometry
    ((3, 20, 20, 4), (1, 3), (1, 2), (0, 0)),            # planes below 4 pixels (generic planar kernel)
])
def test_overlapping_plain_writes_follow_list_order(geom):
    """add=False on overlapping blocks that carry different values: the sequential CPU functor lets the block
    listed last win on every shared pixel (sparse_gather.cc:105-129).  Shuffled lists, a block listed twice,
    both stack layouts, the in-place and the copying op, host and device count."""
    (N, H, W, C), bs, bst, bo = geom
    rng = np.random.default_rng(H * 7 + C)
    bc = bcount_covering(H, W, bst, bo)
    cells = [(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1]) if rng.random() < 0.7]
    idx = np.array(cells + cells[:3], np.int16)   # three blocks appear twice, with different stack rows
    rng.shuffle(idx, axis=0)
    M = len(idx)
    cnt = np.array([M], np.int32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    idxd = dev(idx)
    dcount = torch.tensor([M - 2], dtype=torch.int32, device=DEV)
    for transpose in (False, True):
        shape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
        stack = rng.standard_normal(shape).astype(np.float32)
        y_o = orc.sparse_scatter(stack, cnt, idx, base, bs, bst, bo, add=False, transpose=transpose)
        assert not np.array_equal(y_o, orc.sparse_scatter(stack[::-1].copy(), cnt, idx[::-1].copy(), base, bs, bst, bo,
                                                          add=False, transpose=transpose)), "order must matter here"
        sd = dev(stack)
        y = sbnet_amd.sparse_scatter(sd, cnt, idxd, dev(base), bs, bst, bo, add=False, transpose=transpose)
        np.testing.assert_array_equal(host(y), y_o)
        yv = dev(base)
        sbnet_amd.sparse_scatter_var(sd, cnt, idxd, yv, bs, bst, bo, add=False, transpose=transpose)
        np.testing.assert_array_equal(host(yv), y_o)
        if (transpose or M <= 192) and bs[0] <= 2 * bst[0] and bs[1] <= 2 * bst[1] and bs[0] * bs[1] >= 4:
            # at most 2x2 blocks over a pixel (and, for an NHWC stack, at most 192 blocks): the in-place op needs no
            # scratch for the order (the kernel compares the list itself; lists longer than a workgroup's first
            # fetch included)
            yv = dev(base)
            ops.scatter_forward(sd, cnt, idxd, yv, bs, bst, bo, False, False, transpose, use_var=True, scratch=False)
            np.testing.assert_array_equal(host(yv), y_o)
            yv = dev(base)
            ops.scatter_forward(sd, dcount, idxd, yv, bs, bst, bo, False, False, transpose, use_var=True, scratch=False)
            np.testing.assert_array_equal(host(yv), orc.sparse_scatter(stack, [M - 2], idx, base, bs, bst, bo, add=False,
                                                                        transpose=transpose))
        # the count on the device: the last two rows of the list do not take part
        y_o2 = orc.sparse_scatter(stack, [M - 2], idx, base, bs, bst, bo, add=False, transpose=transpose)
        yv = dev(base)
        sbnet_amd.sparse_scatter_var(sd, dcount, idxd, yv, bs, bst, bo, add=False, transpose=transpose)
        np.testing.assert_array_equal(host(yv), y_o2)
        y = sbnet_amd.sparse_scatter(sd, dcount, idxd, dev(base), bs, bst, bo, add=False, transpose=transpose)
        np.testing.assert_array_equal(host(y), y_o2)


def test_overlapping_plain_writes_large_enough_for_the_one_pass_copy():
    """The copying op on 16 MB or more of blocks builds its output from uncovered pixels (copied) and covered
    ones (scattered); with overlapping plain writes both parts are told apart by the owner map."""
    rng = np.random.default_rng(5)
    N, H, W, C = 1, 256, 256, 64
    bs, bst, bo = (18, 18), (16, 16), (-1, -1)
    bc = bcount_covering(H, W, bst, bo)
    cells = [(0, i, j) for i in range(bc[0]) for j in range(bc[1]) if rng.random() < 0.8]
    idx = np.array(cells, np.int16)
    rng.shuffle(idx, axis=0)
    M = len(idx)
    assert M * bs[0] * bs[1] * C * 4 >= (16 << 20)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    for transpose in (False, True):
        shape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
        stack = rng.standard_normal(shape).astype(np.float32)
        y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=False, transpose=transpose)
        y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=False, transpose=transpose)
        np.testing.assert_array_equal(host(y), y_o)


@pytest.mark.parametrize("geom", [((63, 63), 32), ((65, 65), 32), ((31, 31), 33), ((127, 127), 16), ((63, 63), 18)])
def test_planar_scatter_short_last_split(geom):
    """Block planes whose split into tiles leaves 1-3 pixels for the last tile (63x63 = 31*128 + 1 pixels with
    32 channels): the transposed scatter moves that tail float by float; every mode against the oracle."""
    (R, S), C = geom
    rng = np.random.default_rng(R * S + C)
    N, H, W = 1, R + 9, 2 * S + 5
    bs, bst, bo = (R, S), (R, S), (-3, -2)
    idx = np.array([(0, 0, 0), (0, 0, 1), (0, 1, 0), (0, 1, 2)], np.int16)
    M = len(idx)
    stack = rng.integers(-8, 9, size=(M, C, R, S)).astype(np.float32)
    base = rng.integers(-4, 5, size=(N, H, W, C)).astype(np.float32)
    g_o = orc.sparse_gather(base, [M], idx, bs, bst, bo, transpose=True)
    g = sbnet_amd.sparse_gather(dev(base), [M], dev(idx), bs, bst, bo, transpose=True)
    np.testing.assert_array_equal(host(g), g_o)
    for add, atomic in ((False, False), (True, False), (True, True)):
        y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=add, atomic=atomic, transpose=True)
        yv = dev(base)
        sbnet_amd.sparse_scatter_var(dev(stack), [M], dev(idx), yv, bs, bst, bo, add=add, atomic=atomic, transpose=True)
        np.testing.assert_array_equal(host(yv), y_o, err_msg="add %s atomic %s" % (add, atomic))


def test_overlapping_add_with_repeated_blocks_falls_back_to_atomics():
    rng = np.random.default_rng(77)
    N, H, W, C = 1, 24, 24, 8
    bs, bst, bo = (8, 8), (4, 4), (0, 0)
    idx = np.array([(0, 1, 1), (0, 2, 2), (0, 1, 1), (0, 1, 2), (0, 2, 2)], np.int16)  # two blocks listed twice
    M = len(idx)
    stack = rng.standard_normal((M, 8, 8, C)).astype(np.float32)
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True)
    mag = orc.sparse_scatter(np.abs(stack), [M], idx, np.abs(base), bs, bst, bo, add=True, atomic=True)
    y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=True, atomic=True)
    assert_atomic_close(host(y), y_o, mag)


def test_overlapping_add_many_blocks_per_pixel_uses_atomics():
    rng = np.random.default_rng(78)
    N, H, W, C = 2, 20, 20, 4
    bs, bst, bo = (9, 9), (2, 2), (-3, -3)   # up to 5x5 blocks cover a pixel
    bc = bcount_covering(H, W, bst, bo)
    idx = np.array([(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1])], np.int16)
    M = len(idx)
    stack = rng.standard_normal((M, 9, 9, C)).astype(np.float32)
    base = np.zeros((N, H, W, C), np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True)
    mag = orc.sparse_scatter(np.abs(stack), [M], idx, base, bs, bst, bo, add=True, atomic=True)
    y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=True, atomic=True)
    err = np.abs(host(y).astype(np.float64) - y_o)
    assert (err <= 1e-5 * mag + 1e-30).all()   # up to 25 addends per pixel: 2*24*2^-24 = 3e-6 of the magnitude


@pytest.mark.parametrize("geom", [
    # (N, H, W, C), bsize, bstride, boffset, transpose
    ((2, 40, 52, 8), (6, 6), (3, 3), (-2, -1), True),        # planar stack, 2x2 blocks per pixel: 4 passes
    ((1, 120, 130, 32), (27, 27), (25, 25), (-1, -1), True),  # the BEV geometry (2-pixel seams)
    ((2, 33, 47, 4), (5, 7), (2, 3), (-2, -3), True),        # 3x3 blocks per pixel: 9 passes
    ((2, 33, 47, 4), (5, 7), (2, 3), (-2, -3), False),       # NHWC stack beyond the owner-computes limit
    ((1, 30, 30, 8), (8, 8), (2, 2), (0, 0), False),         # 4x4 blocks per pixel: 16 passes
    ((1, 30, 30, 12), (6, 6), (4, 4), (3, 2), True),         # positive offset: blocks at -1 reach into the image
])
def test_overlapping_add_in_passes(geom):
    """add=True, atomic=True where the owner-computes kernel does not apply runs as passes of plain adds over
    classes of non-overlapping blocks: exact for integer data, within the atomic bar for real data, and
    bit-reproducible from run to run."""
    (N, H, W, C), bs, bst, bo, transpose = geom
    rng = np.random.default_rng(H + C)
    lo = (-(-(bs[0] - 1 + bo[0]) // bst[0]) if bo[0] > 0 else 0, -(-(bs[1] - 1 + bo[1]) // bst[1]) if bo[1] > 0 else 0)
    bc = bcount_covering(H, W, bst, bo)
    cells = [(n, i, j) for n in range(N) for i in range(-lo[0], bc[0]) for j in range(-lo[1], bc[1])
             if rng.random() < 0.7]
    idx = np.array(cells, np.int16)
    rng.shuffle(idx, axis=0)
    M = len(idx)
    shape = (M, C, bs[0], bs[1]) if transpose else (M, bs[0], bs[1], C)
    base = rng.integers(-4, 5, size=(N, H, W, C)).astype(np.float32)
    stack = rng.integers(-8, 9, size=shape).astype(np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True, transpose=transpose)
    y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=True, atomic=True,
                                 transpose=transpose)
    np.testing.assert_array_equal(host(y), y_o)
    stack = rng.standard_normal(shape).astype(np.float32) * np.float32(10.0) ** rng.integers(-3, 4, size=shape)
    stack = stack.astype(np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True, transpose=transpose)
    mag = orc.sparse_scatter(np.abs(stack), [M], idx, np.abs(base), bs, bst, bo, add=True, atomic=True,
                             transpose=transpose)
    runs = []
    for _ in range(3):
        yd = dev(base)
        sbnet_amd.sparse_scatter_var(dev(stack), [M], dev(idx), yd, bs, bst, bo, add=True, atomic=True,
                                     transpose=transpose)
        runs.append(host(yd))
    err = np.abs(runs[0].astype(np.float64) - y_o.astype(np.float64))
    assert (err <= 2e-6 * mag.astype(np.float64) + 1e-30).all()   # up to 16 addends: 2*15*2^-24 = 1.8e-6
    assert runs[0].tobytes() == runs[1].tobytes() == runs[2].tobytes()


def test_overlapping_add_in_passes_with_repeated_blocks():
    """A block listed twice makes two workgroups of one pass add to the same pixels; the duplicate check then
    routes the whole call through hardware atomics."""
    rng = np.random.default_rng(5)
    N, H, W, C = 1, 24, 24, 8
    bs, bst, bo = (6, 6), (3, 3), (0, 0)
    bc = bcount_covering(H, W, bst, bo)
    idx = np.array([(0, i, j) for i in range(bc[0]) for j in range(bc[1])] * 2, np.int16)
    M = len(idx)
    stack = rng.integers(-8, 9, size=(M, C, 6, 6)).astype(np.float32)
    base = np.zeros((N, H, W, C), np.float32)
    y_o = orc.sparse_scatter(stack, [M], idx, base, bs, bst, bo, add=True, atomic=True, transpose=True)
    y = sbnet_amd.sparse_scatter(dev(stack), [M], dev(idx), dev(base), bs, bst, bo, add=True, atomic=True,
                                 transpose=True)
    np.testing.assert_array_equal(host(y), y_o)


@pytest.mark.parametrize("geom", [
    # (N, H, W, C), bsize, bstride, boffset
    ((2, 40, 52, 8), (6, 6), (6, 6), (-2, -1)),            # tiling
    ((2, 40, 52, 8), (6, 6), (3, 3), (-2, -1)),            # overlapping 2x2: owner-computes add / passes
    ((1, 120, 130, 32), (27, 27), (25, 25), (-1, -1)),     # planes split over tiles (line-owning gather)
    ((3, 20, 20, 4), (1, 3), (1, 3), (0, 0)),              # planes below 4 pixels (generic planar kernel)
    ((1, 30, 30, 6), (7, 7), (2, 2), (0, 0)),              # 4x4 blocks per pixel, 2-channel vectors
])
def test_device_resident_count(geom):
    """reduce_mask(sync=False) leaves the count on the GPU; gather and scatter given that tensor read it there,
    are launched for the whole list capacity and must touch only the first `count` blocks."""
    (N, H, W, C), bs, bst, bo = geom
    rng = np.random.default_rng(C * 100 + H)
    bc = bcount_covering(H, W, bst, bo)
    # isolated mask pixels at a rate that leaves about half of the blocks active
    mask = (rng.random((N, H, W, 1)) < 1.0 - 0.5 ** (1.0 / (bs[0] * bs[1]))).astype(np.float32)
    x = rng.integers(-8, 9, size=(N, H, W, C)).astype(np.float32)
    tol = 0.5
    idx_o, cnt_o = orc.reduce_mask(mask, bc, bs, bst, bo, tol, False)
    M, cap = int(cnt_o[0]), N * bc[0] * bc[1]
    assert 0 < M < cap
    r = sbnet_amd.reduce_mask(dev(mask), bc, bs, bst, bo, tol=tol, avgpool=False, sync=False)
    assert r.bin_counts.is_cuda
    overlap = bst[0] < bs[0] or bst[1] < bs[1]
    xd = dev(x)
    for transpose in (False, True):
        g_o = orc.sparse_gather(x, cnt_o, idx_o, bs, bst, bo, transpose=transpose)
        shape = (cap,) + g_o.shape[1:]
        out = torch.full(shape, 555.0, dtype=torch.float32, device=DEV)
        g = sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, bs, bst, bo, transpose=transpose,
                                    out=out)
        assert tuple(g.shape) == shape
        np.testing.assert_array_equal(host(g[:M]), g_o)
        assert float(g[M:].min()) == 555.0 and float(g[M:].max()) == 555.0
        # rows of the stack past the count hold values that must not reach the tensor
        g[M:] = 1.0e6
        base = rng.integers(-4, 5, size=(N, H, W, C)).astype(np.float32)
        for add, atomic in ((False, False), (True, True)) if overlap else ((False, False), (True, False), (True, True)):
            y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, base, bs, bst, bo, add=add, atomic=atomic,
                                     transpose=transpose)
            y = sbnet_amd.sparse_scatter(g, r.bin_counts, r.active_block_indices, dev(base), bs, bst, bo, add=add,
                                         atomic=atomic, transpose=transpose)
            np.testing.assert_array_equal(host(y), y_o)
            yv = dev(base)
            sbnet_amd.sparse_scatter_var(g, r.bin_counts, r.active_block_indices, yv, bs, bst, bo, add=add,
                                         atomic=atomic, transpose=transpose)
            np.testing.assert_array_equal(host(yv), y_o)


def test_whole_pipeline_in_a_hip_graph():
    """reduce_mask -> gather -> scatter_var captured once and replayed on different masks and inputs: with the
    count on the device nothing in the pipeline waits for the host, and every replay must match the oracle."""
    rng = np.random.default_rng(99)
    N, H, W, C = 1, 120, 130, 32
    bs, bst, bo = (27, 27), (25, 25), (-1, -1)
    bc = bcount_covering(H, W, bst, bo)
    cap = N * bc[0] * bc[1]
    mask_s = torch.zeros((N, H, W, 1), device=DEV)
    x_s = torch.zeros((N, H, W, C), device=DEV)
    y_s = torch.zeros((N, H, W, C), device=DEV)
    stack_s = torch.zeros((cap, C, bs[0], bs[1]), device=DEV)

    def pipeline():
        r = sbnet_amd.reduce_mask(mask_s, bc, bs, bst, bo, tol=0.5, avgpool=False, sync=False)
        sbnet_amd.sparse_gather(x_s, r.bin_counts, r.active_block_indices, bs, bst, bo, transpose=True, out=stack_s)
        sbnet_amd.sparse_scatter_var(stack_s, r.bin_counts, r.active_block_indices, y_s, bs, bst, bo, add=False,
                                     transpose=True)
        return r

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pipeline()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        r = pipeline()
    for rep in range(4):
        mask = (rng.random((N, H, W, 1)) < 0.0008 * (rep + 1)).astype(np.float32)
        x = rng.standard_normal((N, H, W, C)).astype(np.float32)
        mask_s.copy_(dev(mask))
        x_s.copy_(dev(x))
        y_s.fill_(-3.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        idx_o, cnt_o = orc.reduce_mask(mask, bc, bs, bst, bo, 0.5, False)
        M = int(cnt_o[0])
        assert int(r.bin_counts.cpu()[0]) == M
        np.testing.assert_array_equal(host(r.active_block_indices)[:M], idx_o[:M])
        g_o = orc.sparse_gather(x, cnt_o, idx_o, bs, bst, bo, transpose=True)
        np.testing.assert_array_equal(host(stack_s[:M]), g_o)
        y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, np.full_like(x, -3.0), bs, bst, bo, add=False, transpose=True)
        np.testing.assert_array_equal(host(y_s), y_o)


@pytest.mark.parametrize("seed", range(32))
def test_random_geometries(seed):
    """Seeded random block geometries (sizes, strides, offsets on either side of zero, channel counts of every
    vector width, partial channel chunks, planes from 1 to ~1200 pixels), random block lists in random order
    with off-image and out-of-range rows: every op and mode against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(6):
        N = int(rng.integers(1, 4))
        C = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 20, 32, 36, 48, 64, 68]))
        R, S = int(rng.integers(1, 36)), int(rng.integers(1, 36))
        U = int(rng.integers(max(1, R // 2), R + 3))
        V = int(rng.integers(max(1, S // 2), S + 3))
        H, W = int(rng.integers(R, 3 * R + 20)), int(rng.integers(S, 3 * S + 20))
        bo = (int(rng.integers(-R + 1, 3)), int(rng.integers(-S + 1, 3)))
        bc = bcount_covering(H, W, (U, V), bo)
        cells = [(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1]) if rng.random() < 0.6]
        cells += [(0, 0, 0), (N - 1, bc[0] - 1, bc[1] - 1)]
        cells = sorted(set(cells))
        idx = np.array(cells, np.int16)
        rng.shuffle(idx, axis=0)
        M = len(idx)
        cnt = np.array([M], np.int32)
        bs, bst = (R, S), (U, V)
        tag = "seed %d case %d: N%d H%d W%d C%d bs %s bst %s bo %s M %d" % (seed, case, N, H, W, C, bs, bst, bo, M)
        x = rng.integers(-8, 9, size=(N, H, W, C)).astype(np.float32)
        base = rng.integers(-4, 5, size=(N, H, W, C)).astype(np.float32)
        overlap = U < R or V < S
        xd, idxd = dev(x), dev(idx)
        for transpose in (False, True):
            g_o = orc.sparse_gather(x, cnt, idx, bs, bst, bo, transpose=transpose)
            g = sbnet_amd.sparse_gather(xd, cnt, idxd, bs, bst, bo, transpose=transpose)
            np.testing.assert_array_equal(host(g), g_o, err_msg=tag)
            stack = rng.integers(-8, 9, size=g_o.shape).astype(np.float32)
            sd = dev(stack)
            # (plain writes of overlapping blocks with different values: the block listed last wins)
            modes = [(False, False), (True, True)] if overlap else [(False, False), (True, False), (True, True)]
            for add, atomic in modes:
                y_o = orc.sparse_scatter(stack, cnt, idx, base, bs, bst, bo, add=add, atomic=atomic,
                                         transpose=transpose)
                yv = dev(base)
                sbnet_amd.sparse_scatter_var(sd, cnt, idxd, yv, bs, bst, bo, add=add, atomic=atomic,
                                             transpose=transpose)
                np.testing.assert_array_equal(host(yv), y_o, err_msg=tag + " add %s atomic %s T %s" %
                                              (add, atomic, transpose))
            if overlap:
                # plain writes of identical values: order-free
                y_o = orc.sparse_scatter(g_o, cnt, idx, base, bs, bst, bo, add=False, transpose=transpose)
                y = sbnet_amd.sparse_scatter(g, cnt, idxd, dev(base), bs, bst, bo, add=False, transpose=transpose)
                np.testing.assert_array_equal(host(y), y_o, err_msg=tag)


@pytest.mark.parametrize("seed", range(16))
def test_random_geometries_with_repeated_rows_and_device_counts(seed):
    """The same kind of sweep with what the first one leaves out: lists that name blocks twice, counts that stay on
    the device and stop short of the list, strides down to a third of the block (up to 3x3 blocks over a pixel),
    and both the in-place and the copying op in every mode."""
    for case in range(8):
        rng = np.random.default_rng(50000 + 8 * seed + case)
        N = int(rng.integers(1, 4))
        C = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 20, 32, 36, 48, 64, 68, 128]))
        R, S = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        U = int(rng.integers(max(1, R // 3), R + 3))
        V = int(rng.integers(max(1, S // 3), S + 3))
        H, W = int(rng.integers(R, 3 * R + 20)), int(rng.integers(S, 3 * S + 20))
        bo = (int(rng.integers(-R + 1, 3)), int(rng.integers(-S + 1, 3)))
        bc = bcount_covering(H, W, (U, V), bo)
        cells = [(n, i, j) for n in range(N) for i in range(bc[0]) for j in range(bc[1]) if rng.random() < 0.6]
        cells = sorted(set(cells + [(0, 0, 0), (N - 1, bc[0] - 1, bc[1] - 1)]))
        dups = bool(rng.random() < 0.3)
        if dups:
            cells = cells + cells[:max(1, len(cells) // 5)]
        idx = np.array(cells, np.int16)
        rng.shuffle(idx, axis=0)
        M = len(idx)
        on_device = bool(rng.random() < 0.4)
        Mc = int(rng.integers(1, M + 1)) if on_device else M
        bin_counts = torch.tensor([Mc], dtype=torch.int32, device=DEV) if on_device else np.array([M], np.int32)
        cnt_o = np.array([Mc], np.int32)
        bs, bst = (R, S), (U, V)
        tag = "seed %d case %d: N%d H%d W%d C%d bs %s bst %s bo %s M %d count %d repeats %s on device %s" % (
            seed, case, N, H, W, C, bs, bst, bo, M, Mc, dups, on_device)
        x = rng.integers(-8, 9, size=(N, H, W, C)).astype(np.float32)
        base = rng.integers(-4, 5, size=(N, H, W, C)).astype(np.float32)
        overlap = U < R or V < S
        xd, idxd = dev(x), dev(idx)
        for transpose in (False, True):
            g_o = orc.sparse_gather(x, cnt_o, idx, bs, bst, bo, transpose=transpose)
            shape = (M, C, R, S) if transpose else (M, R, S, C)
            out = torch.full(shape, 7.0, device=DEV) if on_device else None
            g = sbnet_amd.sparse_gather(xd, bin_counts, idxd, bs, bst, bo, transpose=transpose, out=out)
            np.testing.assert_array_equal(host(g)[:Mc], g_o, err_msg=tag)
            if on_device and Mc < M:
                assert float(g[Mc:].min()) == 7.0 and float(g[Mc:].max()) == 7.0, tag   # rows past the count untouched
            stack = rng.integers(-8, 9, size=shape).astype(np.float32)
            sd = dev(stack)
            modes = [(False, False), (True, True)] if (overlap or dups) else [(False, False), (True, False), (True, True)]
            for add, atomic in modes:
                if dups and not overlap and not add:
                    continue   # repeated rows of tiling blocks, plain writes: the library orders overlapping geometries only
                y_o = orc.sparse_scatter(stack[:Mc], cnt_o, idx, base, bs, bst, bo, add=add, atomic=atomic,
                                         transpose=transpose)
                what = tag + " add %s atomic %s transpose %s" % (add, atomic, transpose)
                yv = dev(base)
                sbnet_amd.sparse_scatter_var(sd, bin_counts, idxd, yv, bs, bst, bo, add=add, atomic=atomic,
                                             transpose=transpose)
                np.testing.assert_array_equal(host(yv), y_o, err_msg=what + " (in place)")
                y = sbnet_amd.sparse_scatter(sd, bin_counts, idxd, dev(base), bs, bst, bo, add=add, atomic=atomic,
                                             transpose=transpose)
                np.testing.assert_array_equal(host(y), y_o, err_msg=what + " (copying)")


# ---------------------------------------------------------------------------------------------
# functor-level entry points and the copy
# ---------------------------------------------------------------------------------------------

def test_reference_functors_in_cxx_against_the_oracle():
    """tests/cxx/functor_shim_gpu.cpp drives reduce_mask -> sparse_gather -> copy + sparse_scatter through the
    reference's functor templates, specialised by include/sbnet_reference_functors.hpp, and compares every result
    with the CPU oracle bit for bit.  The program is built beforehand (make -C tests/cxx, part of build())."""
    import subprocess
    exe = os.path.join(HERE, "cxx", "_build", "functor_shim_gpu")
    assert os.path.exists(exe), "tests/cxx/_build/functor_shim_gpu is missing: run make -C tests/cxx"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "functor shim gpu ok" in out.stdout


def test_functor_level_entry_points():
    import ctypes
    from sbnet_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(31)
    N, H, W, C = 2, 30, 40, 12
    R, S, U, V, oh, ow = 7, 5, 6, 5, -2, -1
    bc = bcount_covering(H, W, (U, V), (oh, ow))
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    mask = rng.standard_normal((N, H, W, 1)).astype(np.float32)
    idx_o, cnt_o = orc.reduce_mask(mask, bc, (R, S), (U, V), (oh, ow), 0.5, False)
    M = int(cnt_o[0])
    idx_d = dev(idx_o)
    xd = dev(x)
    for transpose in (0, 1):
        g_o = orc.sparse_gather(x, cnt_o, idx_o, (R, S), (U, V), (oh, ow), transpose=bool(transpose))
        g = torch.empty(g_o.shape, dtype=torch.float32, device=DEV)
        assert L.sbnet_sparse_gather_functor(xd.data_ptr(), N, H, W, C, g.data_ptr(), oh, ow, R, S, U, V, M,
                                             idx_d.data_ptr(), transpose, None) == 0
        np.testing.assert_array_equal(host(g), g_o)
        base = rng.standard_normal((N, H, W, C)).astype(np.float32)
        yd = dev(base)
        assert L.sbnet_sparse_scatter_functor(g.data_ptr(), N, H, W, C, yd.data_ptr(), oh, ow, R, S, U, V, M,
                                              idx_d.data_ptr(), 1, transpose, 1, None) == 0
        y_o = orc.sparse_scatter(g_o, cnt_o, idx_o, base, (R, S), (U, V), (oh, ow), add=True, atomic=True,
                                 transpose=bool(transpose))
        mag = orc.sparse_scatter(np.abs(g_o), cnt_o, idx_o, np.abs(base), (R, S), (U, V), (oh, ow), add=True,
                                 atomic=True, transpose=bool(transpose))
        assert_atomic_close(host(yd), y_o, mag)
    for count in (0, 1, 3, 4, 1023, 4096 + 5):
        src = torch.arange(count + 3, dtype=torch.float32, device=DEV)
        dst = torch.full((count + 3,), -1.0, device=DEV)
        for off in (0, 1):
            dst.fill_(-1.0)
            assert L.sbnet_copy_tensor(dst.data_ptr() + 4 * off, src.data_ptr() + 4 * off, count, None) == 0
            torch.cuda.synchronize()
            assert torch.equal(dst[off:off + count], src[off:off + count])
            assert float(dst[off + count:].max()) == -1.0


# ---------------------------------------------------------------------------------------------
# the five benchmark configurations at full size
# ---------------------------------------------------------------------------------------------

def run_workload(wl, base=None):
    """reduce_mask -> gather -> (centre crop) -> scatter on a Workload, compared op by op."""
    idx_o, cnt_o, r = check_reduce(wl.mask, wl.bcount, wl.bsize, wl.bstride, wl.boffset, wl.tol, wl.avgpool)
    M = int(cnt_o[0])
    xd = dev(wl.x)
    g = sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, wl.bsize, wl.bstride, wl.boffset,
                                transpose=wl.transpose)
    g_o = orc.sparse_gather(wl.x, cnt_o, idx_o, wl.bsize, wl.bstride, wl.boffset, transpose=wl.transpose, omp=True)
    np.testing.assert_array_equal(host(g), g_o)
    q = workloads.centre_crop(g, wl.bsize, wl.s_bsize, wl.transpose).contiguous()
    q_o = np.ascontiguousarray(workloads.centre_crop(g_o, wl.bsize, wl.s_bsize, wl.transpose))
    if base is None:
        base = np.zeros(wl.shape, np.float32) if wl.name == "C1" else wl.x
    fn = sbnet_amd.sparse_scatter_var if wl.s_var else sbnet_amd.sparse_scatter
    bd = dev(base)
    y = fn(q, r.bin_counts, r.active_block_indices, bd, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=wl.s_add,
           atomic=wl.s_atomic, transpose=wl.transpose)
    y_o = orc.sparse_scatter(q_o, cnt_o, idx_o, base, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=wl.s_add,
                             atomic=wl.s_atomic, transpose=wl.transpose)
    np.testing.assert_array_equal(host(y), y_o)
    if wl.s_var and not wl.s_add:
        # the in-place write as a C-ABI caller without scratch gets it (what bench.py times): the overlapping
        # rows and columns of neighbouring blocks carry the same values here, so no order is needed
        from sbnet_amd import ops
        bd2 = dev(base)
        ops.scatter_forward(q, r.bin_counts, r.active_block_indices, bd2, wl.s_bsize, wl.s_bstride, wl.s_boffset,
                            wl.s_add, wl.s_atomic, wl.transpose, use_var=True, scratch=False)
        np.testing.assert_array_equal(host(bd2), y_o)
    return M


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("size", workloads.REFERENCE_LAYER_SIZES, ids=str)
def test_reference_layer_sizes(size, transpose):
    """The three shapes the reference's test times its ops on (benchmarkLayerSizes, test_sparse_blocks.py:440-443):
    18x18 blocks at stride 18, offset (-1,-2), every block active, copying scatter onto a base of 10.0
    (test_sparse_blocks.py:161, 228), full size, op by op against the oracle."""
    wl = workloads.reference_layer(size, transpose)
    M = run_workload(wl, base=np.full(wl.shape, 10.0, np.float32))
    assert M == wl.bcount[0] * wl.bcount[1]


def test_config1_plumbing():
    c = GOLD["config1"]
    wl = workloads.config1(c["seed"])
    assert run_workload(wl) == len(c["expected_indices"])


def test_config2_ellipses_avgpool(kernel_path):
    assert run_workload(workloads.config2()) > 10


@pytest.mark.parametrize("density", [0.05, 0.15, 0.30])
def test_config3_bev(density, kernel_path):
    wl = workloads.config3(density)
    M = run_workload(wl)
    assert abs(M / 1024.0 - density) < 0.03


def test_config3_roundtrip_is_identity(kernel_path):
    """scatter_var(gather(x)) with the gather geometry rewrites x with its own values: x is unchanged,
    and scattering into zeros reproduces x exactly on the covered pixels (size-independent property)."""
    wl = workloads.config3(0.30)
    xd = dev(wl.x)
    r = sbnet_amd.reduce_mask(dev(wl.mask), wl.bcount, wl.bsize, wl.bstride, wl.boffset, tol=wl.tol)
    g = sbnet_amd.sparse_gather(xd, r.bin_counts, r.active_block_indices, wl.bsize, wl.bstride, wl.boffset,
                                transpose=True)
    keep = xd.clone()
    sbnet_amd.sparse_scatter_var(g, r.bin_counts, r.active_block_indices, xd, wl.bsize, wl.bstride, wl.boffset,
                                 add=False, transpose=True)
    assert torch.equal(xd, keep)
    z = torch.zeros_like(xd)
    sbnet_amd.sparse_scatter_var(g, r.bin_counts, r.active_block_indices, z, wl.bsize, wl.bstride, wl.boffset,
                                 add=False, transpose=True)
    covered = z != 0
    assert torch.equal(z[covered], xd[covered]) and 0.2 < float(covered.float().mean()) < 0.45


def test_config4_overlapping_atomic_add():
    wl = workloads.config4()
    N, H, W, C = wl.shape
    M = len(wl.indices)
    gen = torch.Generator(device=DEV).manual_seed(1004)
    stack = torch.rand((M, 16, 16, C), generator=gen, device=DEV) * 2.0 - 1.0
    base = torch.zeros((N, H, W, C), device=DEV)
    idx_d = dev(wl.indices)
    out = sbnet_amd.sparse_scatter_var(stack, [M], idx_d, base, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                                       atomic=True)
    assert out.data_ptr() == base.data_ptr()
    y_o = np.zeros((N, H, W, C), np.float32)
    orc.sparse_scatter_raw(host(stack), M, wl.indices, y_o, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                           transpose=False)
    # the Python mirror passes scratch, so the adds run without atomics in the CPU functor's order: exact
    np.testing.assert_array_equal(host(base), y_o)
    # second pass on top of the first, still against the sequential oracle
    sbnet_amd.sparse_scatter_var(stack, [M], idx_d, base, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                                 atomic=True)
    orc.sparse_scatter_raw(host(stack), M, wl.indices, y_o, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                           transpose=False)
    np.testing.assert_array_equal(host(base), y_o)
    # the same through the raw ABI without scratch: hardware atomics, equal to rounding
    import ctypes
    from sbnet_amd import _lib
    L = _lib.load()
    I2 = ctypes.c_int32 * 2
    base2 = torch.zeros((N, H, W, C), device=DEV)
    rc = L.sbnet_sparse_scatter_var(stack.data_ptr(), M, idx_d.data_ptr(), base2.data_ptr(),
                                    (ctypes.c_int64 * 4)(N, H, W, C), 4, I2(16, 16), 2, I2(8, 8), 2, I2(0, 0), 2, 1, 1, 0,
                                    None, 0, None)
    assert rc == 0
    y1 = np.zeros((N, H, W, C), np.float32)
    orc.sparse_scatter_raw(host(stack), M, wl.indices, y1, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                           transpose=False)
    mag = np.zeros((N, H, W, C), np.float32)
    orc.sparse_scatter_raw(np.abs(host(stack)), M, wl.indices, mag, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=True,
                           transpose=False)
    assert_atomic_close(host(base2), y1, mag)
    # checksum: every in-image stack element lands exactly once (float64 sums agree to rounding)
    ar = torch.arange(16, device=DEV)[None, :]
    rows = (ar + 8 * idx_d[:, 1:2].long()) < H
    cols = (ar + 8 * idx_d[:, 2:3].long()) < W
    inside = (rows[:, :, None] & cols[:, None, :])[..., None]
    assert abs(float(base.double().sum()) - 2.0 * float((stack.double() * inside).sum())) < 1e-3 * M


def test_config5_many_small_images(kernel_path):
    M = run_workload(workloads.config5())
    assert M > 10000
