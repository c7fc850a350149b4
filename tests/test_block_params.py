"""Block-geometry arithmetic (sbnet_amd/block_params.py) against what the reference's tests hold:
benchmark/tf_conv_dims_tests.py:40-46 (output sizes equal a real convolution's), :72-140 (padding
vectors), and the block parameters implied by the known-answer tables of sparse_conv_tests.py."""
import json
import os

import pytest
import torch
import torch.nn.functional as F

from sbnet_amd import block_params as bp

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "known_answers.json")) as f:
    GOLD = json.load(f)


@pytest.mark.parametrize("padding", ["SAME", "VALID"])
@pytest.mark.parametrize("stride", [1, 2, 3])
@pytest.mark.parametrize("ksize", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("insize", [6, 7, 10, 11])
def test_out_size_matches_a_real_convolution(insize, ksize, stride, padding):
    if ksize > insize:
        pytest.skip("kernel larger than input")
    x = torch.ones(1, 1, insize, insize)
    w = torch.ones(1, 1, ksize, ksize)
    out = bp.calc_out_size_1d(insize, ksize, stride, padding)
    if padding == "SAME":
        pad = bp.calc_padding_1d(insize, out, ksize, stride, padding)
        x = F.pad(x, (pad // 2, pad - pad // 2, pad // 2, pad - pad // 2))
    assert F.conv2d(x, w, stride=stride).shape[2] == out


def test_padding_vectors():
    # tf_conv_dims_tests.py:73-81, 122-140
    assert bp.calc_padding_4d([1, 5, 6, 1], [2, 3, 1, 1], [1, 1, 1, 1], "SAME") == (0, 1, 1, 1)
    assert bp.calc_padding_4d([1, 5, 5, 1], [2, 3, 1, 1], [1, 1, 1, 1], "VALID") == (0, 0, 0, 0)
    assert bp.calc_padding_4d([1, 5, 6, 1], [2, 3, 1, 1], [1, 2, 2, 1], "SAME") == (0, 1, 0, 1)


def test_padding_errors():
    # tf_conv_dims_tests.py:83-103: AssertionError with these texts
    with pytest.raises(AssertionError, match="Expect `ksize` a list/tuple of length 4."):
        bp.calc_padding_4d([1, 5, 6, 1], [2, 3, 1, 1, 1], [2, 1, 1, 1], "SAME")
    with pytest.raises(AssertionError, match="Expect first and last dimension of `strides` = 1."):
        bp.calc_padding_4d([1, 5, 6, 1], [2, 3, 1, 1], [2, 1, 1, 1], "SAME")


@pytest.mark.parametrize("case", GOLD["pipeline"], ids=lambda c: c["name"])
def test_block_params_of_known_answer_tables(case):
    H, W = len(case["mask"]), len(case["mask"][0])
    p = bp.calc_block_params([1, H, W, 1], [1] + case["bsize"] + [1], case["ksize"] + [1, 1],
                             [1] + case["conv_strides"] + [1], case["padding"])
    assert p.bsize == case["bsize"] and p.bstrides == case["bstride"] and p.boffset == case["boffset"]
    assert p.bcount == case["bcount"] and p.bsize_out == case["bsize_out"]


def test_block_params_of_benchmark_configs():
    # 3x3 SAME convolution geometry of the benchmark configurations
    p = bp.calc_block_params([1, 64, 64, 16], [1, 10, 10, 1], [3, 3, 1, 1], [1, 1, 1, 1], "SAME")
    assert (p.bstrides, p.boffset, p.bcount, p.bsize_out) == ([8, 8], [-1, -1], [8, 8], [8, 8])
    p = bp.calc_block_params([4, 256, 256, 64], [1, 18, 18, 1], [3, 3, 1, 1], [1, 1, 1, 1], "SAME")
    assert (p.bstrides, p.boffset, p.bcount, p.bsize_out) == ([16, 16], [-1, -1], [16, 16], [16, 16])
    p = bp.calc_block_params([1, 800, 800, 128], [1, 27, 27, 1], [3, 3, 1, 1], [1, 1, 1, 1], "SAME")
    assert (p.bstrides, p.boffset, p.bcount, p.bsize_out) == ([25, 25], [-1, -1], [32, 32], [25, 25])
    p = bp.calc_block_params([64, 128, 128, 32], [1, 6, 6, 1], [3, 3, 1, 1], [1, 1, 1, 1], "SAME")
    assert (p.bstrides, p.boffset, p.bcount, p.bsize_out) == ([4, 4], [-1, -1], [32, 32], [4, 4])
    # residual block 1x1, 3x3, 1x1 has a 3x3 receptive field (sparse_conv_lib.py:417-421)
    q = bp.calc_block_params_res_block([1, 800, 800, 128], [1, 27, 27, 1],
                                       [[1, 1, 128, 32], [3, 3, 32, 32], [1, 1, 32, 128]], [1, 1, 1, 1], "SAME")
    assert q == bp.calc_block_params([1, 800, 800, 128], [1, 27, 27, 1], [3, 3, 1, 1], [1, 1, 1, 1], "SAME")


def test_covering_block_count():
    # sbnet_ops/tests/test_sparse_blocks.py:101-112
    assert bp.calc_block_count_covering(512, 0, 8) == 64
    assert bp.calc_block_count_covering(5, -1, 1) == 6
    assert bp.calc_block_count_covering(2048, -1, 300) == 7
