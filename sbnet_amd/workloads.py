"""Seeded synthetic inputs for the five benchmark configurations of the
reduce_mask -> sparse_gather -> sparse_scatter path (numpy only; used by bench.py and the tests).

Each generator returns a `Workload`: tensor shape, block geometry for reduce_mask / gather and for
scatter, op attributes, and the host arrays (x, mask, or a ready-made block list where the
configuration draws active blocks directly).  Geometry follows the reference's conventions
(block (n,bh,bw) covers rows boffset[0]+bh*bstride[0] ... +bsize[0], README.md:66-67 of the
reference); bcount for convolution-shaped configurations is what
sbnet_amd.block_params.calc_block_params gives for a 3x3 SAME convolution.
"""
import collections

import numpy as np

Workload = collections.namedtuple("Workload", [
    "name", "shape",                       # [N,H,W,C]
    "bsize", "bstride", "boffset", "bcount",  # reduce_mask / gather geometry
    "tol", "avgpool", "transpose",
    "s_bsize", "s_bstride", "s_boffset", "s_add", "s_atomic", "s_var",  # scatter geometry / attributes
    "x", "mask", "indices",                # host arrays; `indices` only where blocks are drawn directly
])


def _wl(**kw):
    kw.setdefault("x", None)
    kw.setdefault("mask", None)
    kw.setdefault("indices", None)
    return Workload(**kw)


def config1(seed=1001):
    """[1,64,64,16] U(-1,1); mask = 8x8 grid of 8x8 tiles, each 1 w.p. 0.5; max-pool tol 0.5;
    10x10 blocks, stride 8, offset -1, 8x8 blocks; gather NHWC, scatter add=False into zeros."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1.0, 1.0, size=(1, 64, 64, 16)).astype(np.float32)
    tiles = (rng.random((8, 8)) < 0.5).astype(np.float32)
    mask = np.kron(tiles, np.ones((8, 8), np.float32)).reshape(1, 64, 64, 1)
    return _wl(name="C1", shape=[1, 64, 64, 16], bsize=[10, 10], bstride=[8, 8], boffset=[-1, -1], bcount=[8, 8],
               tol=0.5, avgpool=False, transpose=False, s_bsize=[10, 10], s_bstride=[8, 8], s_boffset=[-1, -1],
               s_add=False, s_atomic=False, s_var=False, x=x, mask=mask)


def _ellipse_mask(rng, N, H, W, per_image, rmin, rmax):
    yy, xx = np.mgrid[0:H, 0:W].astype(np.float32)
    mask = np.zeros((N, H, W), np.float32)
    for n in range(N):
        for _ in range(per_image):
            cy, cx = rng.uniform(0, H), rng.uniform(0, W)
            ry, rx = rng.uniform(rmin, rmax), rng.uniform(rmin, rmax)
            mask[n][((yy - cy) / ry) ** 2 + ((xx - cx) / rx) ** 2 <= 1.0] = 1.0
    return mask


def config2(seed=1002, with_x=True):
    """[4,256,256,64] N(0,1); mask = union of 6 ellipses per image, extents 10-60 px (semi-axes 5-30, which
    gives the ~10 % pixel density the configuration names; 10-60 px semi-axes would give ~25 %); avg-pool tol 0.5;
    18x18 blocks, stride 16, offset -1; gather transposed; scatter add=True of the 16x16 centre
    (stride 16, offset 0: the output geometry of a VALID 3x3 convolution on the block)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((4, 256, 256, 64), dtype=np.float32) if with_x else None
    mask = _ellipse_mask(rng, 4, 256, 256, 6, 5.0, 30.0).reshape(4, 256, 256, 1)
    return _wl(name="C2", shape=[4, 256, 256, 64], bsize=[18, 18], bstride=[16, 16], boffset=[-1, -1],
               bcount=[16, 16], tol=0.5, avgpool=True, transpose=True, s_bsize=[16, 16], s_bstride=[16, 16],
               s_boffset=[0, 0], s_add=True, s_atomic=False, s_var=False, x=x, mask=mask)


def _stroke(mask, p0, p1, width):
    """Sets pixels within width/2 of the segment p0-p1."""
    H, W = mask.shape
    r = width / 2.0
    y0, y1 = int(max(0, min(p0[0], p1[0]) - r)), int(min(H, max(p0[0], p1[0]) + r + 1))
    x0, x1 = int(max(0, min(p0[1], p1[1]) - r)), int(min(W, max(p0[1], p1[1]) + r + 1))
    if y0 >= y1 or x0 >= x1:
        return
    yy, xx = np.mgrid[y0:y1, x0:x1].astype(np.float32)
    d = np.array([p1[0] - p0[0], p1[1] - p0[1]], np.float32)
    L2 = float(d @ d)
    t = np.clip(((yy - p0[0]) * d[0] + (xx - p0[1]) * d[1]) / L2, 0, 1) if L2 > 0 else np.zeros_like(yy)
    dist2 = (yy - (p0[0] + t * d[0])) ** 2 + (xx - (p0[1] + t * d[1])) ** 2
    mask[y0:y1, x0:x1][dist2 <= r * r] = 1.0


def _active_fraction(mask2d, bsize, bstride, boffset, bcount, tol):
    H, W = mask2d.shape
    act = 0
    for bh in range(bcount[0]):
        h0 = boffset[0] + bh * bstride[0]
        for bw in range(bcount[1]):
            w0 = boffset[1] + bw * bstride[1]
            win = mask2d[max(h0, 0):max(h0 + bsize[0], 0), max(w0, 0):max(w0 + bsize[1], 0)]
            act += bool(win.size and win.max() > tol)
    return act / float(bcount[0] * bcount[1])


def config3(density=0.30, seed=1003, with_x=True):
    """LiDAR-BEV shape [1,800,800,128] N(0,1); mask = road-like band of random polyline strokes (width
    20-40 px, value 1) plus Bernoulli(0.02) speckle; max-pool tol 0.5; 27x27 blocks, stride 25, offset -1,
    32x32 blocks; gather transposed; scatter_var in place, add=False, same geometry.

    `density` is the fraction of the 1024 blocks that end up active: strokes are added until it is
    reached.  The speckle carries values in (0, 0.5), below the threshold: with max pooling over 729-pixel
    blocks a super-threshold 2 % speckle would switch every block on and leave nothing to sweep."""
    rng = np.random.default_rng(seed + int(round(density * 1000)))
    H = W = 800
    bsize, bstride, boffset, bcount = [27, 27], [25, 25], [-1, -1], [32, 32]
    m = np.zeros((H, W), np.float32)
    p = np.array([rng.uniform(0, H), rng.uniform(0, W)])
    heading = rng.uniform(0, 2 * np.pi)
    guard = 0
    while _active_fraction(m, bsize, bstride, boffset, bcount, 0.5) < density and guard < 4000:
        guard += 1
        heading += rng.normal(0, 0.5)
        step = rng.uniform(20, 60)
        q = p + step * np.array([np.sin(heading), np.cos(heading)])
        if not (0 <= q[0] < H and 0 <= q[1] < W):
            p = np.array([rng.uniform(0, H), rng.uniform(0, W)])
            heading = rng.uniform(0, 2 * np.pi)
            continue
        _stroke(m, p, q, rng.uniform(20, 40))
        p = q
    speck = rng.random((H, W)) < 0.02
    m = np.where((m == 0) & speck, rng.uniform(0.01, 0.49, size=(H, W)).astype(np.float32), m).astype(np.float32)
    x = rng.standard_normal((1, H, W, 128), dtype=np.float32) if with_x else None
    return _wl(name="C3@%d%%" % int(round(density * 100)), shape=[1, 800, 800, 128], bsize=bsize, bstride=bstride,
               boffset=boffset, bcount=bcount, tol=0.5, avgpool=False, transpose=True, s_bsize=bsize,
               s_bstride=bstride, s_boffset=boffset, s_add=False, s_atomic=False, s_var=True, x=x,
               mask=m.reshape(1, H, W, 1))


def config4(seed=1004, shape=(2, 512, 512, 256)):
    """Overlapping atomic scatter-add: base [2,512,512,256] zeros; 16x16 blocks, stride 8 (every pixel is
    covered by up to 4 blocks), offset 0, 64x64 blocks per image; each block active w.p. 0.25, drawn
    directly (one Bernoulli per 8x8 cell); the block stack is U(-1,1) and is generated by the caller
    from `indices` (it is as large as the base)."""
    rng = np.random.default_rng(seed)
    N, H, W, C = shape
    bcount = [1 + (H - 1) // 8, 1 + (W - 1) // 8]
    cells = rng.random((N, bcount[0], bcount[1])) < 0.25
    idx = np.ascontiguousarray(np.argwhere(cells), dtype=np.int16)  # argwhere returns a transposed view
    return _wl(name="C4", shape=list(shape), bsize=[16, 16], bstride=[8, 8], boffset=[0, 0], bcount=bcount, tol=0.5,
               avgpool=False, transpose=False, s_bsize=[16, 16], s_bstride=[8, 8], s_boffset=[0, 0], s_add=True,
               s_atomic=True, s_var=True, indices=idx)


def config5(seed=1005, with_x=True):
    """Many small images: [64,128,128,32] U(-1,1); per-image Bernoulli(p_i) on 4x4 cells, p_i ~ U(0.05,0.6);
    avg-pool tol 0.3; 6x6 blocks, stride 4, offset -1, 32x32 blocks; gather transposed; scatter add=True of
    the 4x4 centre (stride 4, offset 0)."""
    rng = np.random.default_rng(seed)
    N, H, W, C = 64, 128, 128, 32
    x = rng.uniform(-1.0, 1.0, size=(N, H, W, C)).astype(np.float32) if with_x else None
    p = rng.uniform(0.05, 0.6, size=(N, 1, 1))
    cells = (rng.random((N, H // 4, W // 4)) < p).astype(np.float32)
    mask = np.kron(cells, np.ones((1, 4, 4), np.float32)).reshape(N, H, W, 1)
    return _wl(name="C5", shape=[N, H, W, C], bsize=[6, 6], bstride=[4, 4], boffset=[-1, -1], bcount=[32, 32],
               tol=0.3, avgpool=True, transpose=True, s_bsize=[4, 4], s_bstride=[4, 4], s_boffset=[0, 0],
               s_add=True, s_atomic=False, s_var=False, x=x, mask=mask)


REFERENCE_LAYER_SIZES = [(300, 480, 64), (600, 960, 64), (300, 480, 256)]


def reference_layer(size, transpose=True, seed=1006, with_x=True):
    """The shapes on which the reference's own test times gather + scatter (benchmarkLayerSizes,
    sbnet_ops/tests/test_sparse_blocks.py:440-443, through runTestForOneSize :139-260 and generateInputs :124-133):
    one image [1,H,W,C], mask and x ~ N(0,1), 18x18 blocks at stride 18, offset (-1,-2), block counts by that
    file's covering rule (:101-121), max pooling with tol = the 70th percentile of x (which leaves every block
    active: some pixel of 324 exceeds it), gather, then the copying scatter with add=False and the same geometry."""
    H, W, C = size
    rng = np.random.default_rng(seed + H + C)
    mask = rng.standard_normal((1, H, W, 1), dtype=np.float32)
    x = rng.standard_normal((1, H, W, C), dtype=np.float32) if with_x else None
    sample = x if x is not None else rng.standard_normal(1 << 20, dtype=np.float32)
    tol = float(np.percentile(sample.reshape(-1)[:1 << 22], 70))
    bsize, bstride, boffset = [18, 18], [18, 18], [-1, -2]
    bcount = [1 + (H - boffset[0] - 1) // bstride[0], 1 + (W - boffset[1] - 1) // bstride[1]]
    return _wl(name="L%dx%dx%d" % size, shape=[1, H, W, C], bsize=bsize, bstride=bstride, boffset=boffset, bcount=bcount,
               tol=tol, avgpool=False, transpose=transpose, s_bsize=bsize, s_bstride=bstride, s_boffset=boffset,
               s_add=False, s_atomic=False, s_var=False, x=x, mask=mask)


def centre_crop(stack, bsize, s_bsize, transpose):
    """Stand-in for the VALID convolution between gather and scatter: keeps the centre s_bsize window of
    every gathered block (numpy or torch)."""
    dh, dw = (bsize[0] - s_bsize[0]) // 2, (bsize[1] - s_bsize[1]) // 2
    if transpose:
        return stack[:, :, dh:dh + s_bsize[0], dw:dw + s_bsize[1]]
    return stack[:, dh:dh + s_bsize[0], dw:dw + s_bsize[1], :]
