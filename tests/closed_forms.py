"""Independent numpy / torch statements of what the three ops compute, used to pin the CPU oracle
(and, through it, the HIP kernels).  Nothing here shares code with oracle/ or with the library.

  reduce_mask   README.md:48-67 of the reference: pool the padded mask per block, threshold, list the
                active blocks in row-major order (how benchmark/reduce_mask_tests.py:32-47 checks it,
                through sparse_conv_lib.py:312-317).
  gather        README.md:86-92: slices of the zero-padded tensor stacked along the batch axis.
  scatter       README.md:119-125: slice assignment / addition per block, in list order.
"""
import numpy as np


def _pad_amounts(H, W, bcount, bsize, bstride, boffset):
    h_end = boffset[0] + bstride[0] * (bcount[0] - 1) + bsize[0]
    w_end = boffset[1] + bstride[1] * (bcount[1] - 1) + bsize[1]
    return max(0, -boffset[0]), max(0, h_end - H), max(0, -boffset[1]), max(0, w_end - W)


def np_reduce_mask(mask, bcount, bsize, bstride, boffset, tol, avgpool):
    """Returns the int16 [M,3] list of active blocks in (n, bh, bw) row-major order (M may be 0).

    avg mode sums in float64, which is exact for the integer-valued masks this is used with, then
    divides and compares in float32 as the op does."""
    m = np.asarray(mask, dtype=np.float32)
    m = m.reshape(m.shape[0], m.shape[1], m.shape[2])
    N, H, W = m.shape
    pt, pb, pl, pr = _pad_amounts(H, W, bcount, bsize, bstride, boffset)
    fill = 0.0 if avgpool else -np.inf
    p = np.pad(m.astype(np.float64), ((0, 0), (pt, pb), (pl, pr)), constant_values=fill)
    out = []
    for n in range(N):
        for bh in range(bcount[0]):
            for bw in range(bcount[1]):
                h0 = boffset[0] + bh * bstride[0] + pt
                w0 = boffset[1] + bw * bstride[1] + pl
                win = p[n, max(h0, 0):max(h0 + bsize[0], 0), max(w0, 0):max(w0 + bsize[1], 0)]
                if avgpool:
                    act = np.float32(win.sum()) / np.float32(bsize[0] * bsize[1]) > np.float32(tol)
                else:
                    act = win.size > 0 and win.max() > np.float32(tol)
                if act:
                    out.append((n, bh, bw))
    return np.asarray(out, dtype=np.int16).reshape(-1, 3)


def np_gather(x, idx, bsize, bstride, boffset, transpose):
    x = np.asarray(x, dtype=np.float32)
    N, H, W, C = x.shape
    R, S = bsize
    idx = np.asarray(idx).reshape(-1, 3).astype(np.int64)
    if len(idx) == 0:
        return np.zeros((0, C, R, S) if transpose else (0, R, S, C), np.float32)
    h0 = boffset[0] + idx[:, 1] * bstride[0]
    w0 = boffset[1] + idx[:, 2] * bstride[1]
    pt, pl = max(0, -int(h0.min())), max(0, -int(w0.min()))
    pb, pr = max(0, int(h0.max()) + R - H), max(0, int(w0.max()) + S - W)
    p = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    y = np.stack([p[n, a + pt:a + pt + R, b + pl:b + pl + S, :] for n, a, b in zip(idx[:, 0], h0, w0)])
    return np.ascontiguousarray(y.transpose(0, 3, 1, 2)) if transpose else y


def np_scatter(xblocks, idx, ybase, bsize, bstride, boffset, add, transpose):
    """Sequential in list order: adds accumulate in that order, plain writes let the last block win."""
    y = np.array(ybase, dtype=np.float32, copy=True)
    N, H, W, C = y.shape
    R, S = bsize
    xb = np.asarray(xblocks, dtype=np.float32)
    if transpose:
        xb = xb.transpose(0, 2, 3, 1)
    for ib, (n, bh, bw) in enumerate(np.asarray(idx).reshape(-1, 3).astype(np.int64)):
        h0 = boffset[0] + bh * bstride[0]
        w0 = boffset[1] + bw * bstride[1]
        ha, hb = max(h0, 0), min(h0 + R, H)
        wa, wb = max(w0, 0), min(w0 + S, W)
        if ha >= hb or wa >= wb:
            continue
        src = xb[ib, ha - h0:hb - h0, wa - w0:wb - w0, :]
        if add:
            y[n, ha:hb, wa:wb, :] += src
        else:
            y[n, ha:hb, wa:wb, :] = src
    return y


def box_sum_valid(p, kh, kw, sh=1, sw=1):
    """VALID convolution with an all-ones [kh,kw,1,1] kernel on an NHWC stack with C == 1."""
    M, R, S, C = p.shape
    oh, ow = (R - kh) // sh + 1, (S - kw) // sw + 1
    q = np.zeros((M, oh, ow, C), np.float32)
    for i in range(oh):
        for j in range(ow):
            q[:, i, j, :] = p[:, i * sh:i * sh + kh, j * sw:j * sw + kw, :].sum(axis=(1, 2))
    return q
