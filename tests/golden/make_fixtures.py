"""Writes tests/golden/known_answers.json.

Run from the repository root:  python tests/golden/make_fixtures.py

Nothing here imports or executes the reference, the CPU oracle or the library.  The hand-written
masks and expected outputs are the data the reference's own tests hold (cited per entry, paths
relative to the reference's sbnet_tensorflow/); expected active-block lists are derived with the
independent numpy closed form of tests/closed_forms.py; block parameters are written out as plain
numbers (they follow from sparse_conv_lib.py:343-397 and are re-derived by test_block_params.py).
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from closed_forms import np_gather, np_reduce_mask, np_scatter  # noqa: E402

MASK_5x5 = [[0, 0, 0, 0, 0],
            [0, 0, 1, 0, 0],
            [1, 0, 0, 0, 0],
            [0, 0, 0, 0, 0],
            [0, 0, 0, 0, 0]]

MASK_8x8 = [[0, 0, 0, 0, 0, 1, 1, 1],
            [0, 0, 0, 0, 0, 1, 1, 1],
            [1, 0, 0, 0, 0, 1, 1, 1],
            [0, 0, 0, 0, 0, 1, 1, 1],
            [0, 0, 0, 0, 0, 1, 1, 1],
            [0, 0, 0, 0, 0, 0, 0, 0],
            [0, 0, 0, 0, 0, 0, 0, 0],
            [0, 0, 0, 0, 0, 0, 0, 0]]

# mask -> gather -> VALID conv with an all-ones kernel on an all-ones input -> scatter (add=False)
# into a zero tensor of the output size.  y_exp counts the in-image pixels of each kernel window on
# active blocks (4 / 6 / 9 at corners / edges / interior for 3x3) and is 0 where no block is active.
# The scatter steps by `s_bstride` output pixels where given, else by `bstride` (equal to bsize_out for a
# convolution of stride 1).
PIPELINE = [
    dict(name="mask_valid_3x3", source="benchmark/sparse_conv_tests.py:197-218",
         mask=MASK_5x5, bsize=[3, 3], ksize=[3, 3], conv_strides=[1, 1], padding="VALID",
         bstride=[1, 1], boffset=[0, 0], bcount=[3, 3], bsize_out=[1, 1],
         y_exp=[[9, 9, 9], [9, 9, 9], [9, 0, 0]]),
    dict(name="mask_same_3x3", source="benchmark/sparse_conv_tests.py:220-243 and 437-460",
         mask=MASK_5x5, bsize=[3, 3], ksize=[3, 3], conv_strides=[1, 1], padding="SAME",
         bstride=[1, 1], boffset=[-1, -1], bcount=[5, 5], bsize_out=[1, 1],
         y_exp=[[0, 6, 6, 6, 0], [6, 9, 9, 9, 0], [6, 9, 9, 9, 0], [6, 9, 0, 0, 0], [0, 0, 0, 0, 0]]),
    dict(name="mask_same_even_block_4x4", source="benchmark/sparse_conv_tests.py:245-268",
         mask=MASK_5x5, bsize=[4, 4], ksize=[3, 3], conv_strides=[1, 1], padding="SAME",
         bstride=[2, 2], boffset=[-1, -1], bcount=[3, 3], bsize_out=[2, 2],
         y_exp=[[4, 6, 6, 6, 0], [6, 9, 9, 9, 0], [6, 9, 9, 9, 0], [6, 9, 9, 9, 0], [0, 0, 0, 0, 0]]),
    # the only table whose convolution has a stride: gather blocks step by bsize - k + stride = 4 input pixels,
    # the 2x2 outputs of a block step by 4 / 2 = 2 output pixels (`s_bstride`); one block at offset -1 covers
    # the whole 5x5 input, and the 3x3 output shows its four windows with 2x2, 2x3, 3x2 and 3x3 in-image pixels
    dict(name="mask_same_even_block_strides_5x5_s2", source="benchmark/sparse_conv_tests.py:270-291",
         mask=MASK_5x5, bsize=[5, 5], ksize=[3, 3], conv_strides=[2, 2], padding="SAME",
         bstride=[4, 4], boffset=[-1, -1], bcount=[1, 1], bsize_out=[2, 2], s_bstride=[2, 2],
         y_exp=[[4, 6, 0], [6, 9, 0], [0, 0, 0]]),
    dict(name="mask_valid_large_block_5x5_k2", source="benchmark/sparse_conv_tests.py:293-321",
         mask=MASK_8x8, bsize=[5, 5], ksize=[2, 2], conv_strides=[1, 1], padding="VALID",
         bstride=[4, 4], boffset=[0, 0], bcount=[2, 2], bsize_out=[4, 4],
         y_exp=[[4, 4, 4, 4, 4, 4, 4]] * 4 + [[0, 0, 0, 0, 4, 4, 4]] * 3),
]

# reduce_mask on the hand-written masks of benchmark/reduce_mask_tests.py:49-82 (tol 0, max pooling);
# the same masks with x = arange drive benchmark/sparse_gather_tests.py:81-122.
REDUCE = [
    dict(name="basic_5x5_same", source="benchmark/reduce_mask_tests.py:49-63", mask=MASK_5x5,
         bsize=[3, 3], bstride=[1, 1], boffset=[-1, -1], bcount=[5, 5], tol=0.0, avgpool=False),
    dict(name="larger_8x8_valid", source="benchmark/reduce_mask_tests.py:65-82", mask=MASK_8x8,
         bsize=[5, 5], bstride=[4, 4], boffset=[0, 0], bcount=[2, 2], tol=0.0, avgpool=False),
    # avg pooling over the same masks: a block is active when more than tol of its full bsize area is set
    dict(name="basic_5x5_same_avg", source="benchmark/reduce_mask_tests.py:54-62 mask, avgpool attribute",
         mask=MASK_5x5, bsize=[3, 3], bstride=[1, 1], boffset=[-1, -1], bcount=[5, 5], tol=0.12, avgpool=True),
    dict(name="larger_8x8_valid_avg", source="benchmark/reduce_mask_tests.py:70-81 mask, avgpool attribute",
         mask=MASK_8x8, bsize=[5, 5], bstride=[4, 4], boffset=[0, 0], bcount=[2, 2], tol=0.3, avgpool=True),
]


def config1_inputs(seed=1001):
    """Benchmark configuration 1: x [1,64,64,16] ~U(-1,1); mask = 8x8 grid of 8x8 tiles, each 1 w.p. 0.5."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1.0, 1.0, size=(1, 64, 64, 16)).astype(np.float32)
    tiles = (rng.random((8, 8)) < 0.5).astype(np.float32)
    mask = np.kron(tiles, np.ones((8, 8), np.float32)).reshape(1, 64, 64, 1)
    return x, mask


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    out = {"reduce_mask": [], "pipeline": PIPELINE, "gather_arange": []}
    for c in REDUCE:
        idx = np_reduce_mask(np.asarray(c["mask"], np.float32)[None, :, :, None], c["bcount"], c["bsize"],
                             c["bstride"], c["boffset"], c["tol"], c["avgpool"])
        e = dict(c)
        e["expected_indices"] = idx.tolist()
        out["reduce_mask"].append(e)
        if not c["avgpool"]:
            m = np.asarray(c["mask"], np.float32)
            x = np.arange(m.size, dtype=np.float32).reshape(1, m.shape[0], m.shape[1], 1)
            y = np_gather(x, idx, c["bsize"], c["bstride"], c["boffset"], False)
            out["gather_arange"].append(dict(name=c["name"], source="benchmark/sparse_gather_tests.py:81-122",
                                             bsize=c["bsize"], bstride=c["bstride"], boffset=c["boffset"],
                                             shape=list(m.shape), indices=idx.tolist(),
                                             expected_blocks=y.reshape(len(idx), -1).tolist()))
    # config 1: digests of the closed-form outputs for the seeded inputs
    x, mask = config1_inputs()
    bs, bst, bo, bc = [10, 10], [8, 8], [-1, -1], [8, 8]
    idx = np_reduce_mask(mask, bc, bs, bst, bo, 0.5, False)
    g = np_gather(x, idx, bs, bst, bo, False)
    y = np_scatter(g, idx, np.zeros_like(x), bs, bst, bo, False, False)
    out["config1"] = dict(seed=1001, x_sha256=sha(x), mask_sha256=sha(mask), bsize=bs, bstride=bst, boffset=bo,
                          bcount=bc, tol=0.5, avgpool=False, expected_indices=idx.tolist(),
                          gather_sha256=sha(g), gather_t_sha256=sha(np_gather(x, idx, bs, bst, bo, True)),
                          scatter_sha256=sha(y))
    with open(os.path.join(HERE, "known_answers.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote known_answers.json:", {k: (len(v) if isinstance(v, list) else "dict") for k, v in out.items()})


if __name__ == "__main__":
    main()
