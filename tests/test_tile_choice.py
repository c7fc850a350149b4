"""Host-side launch configuration of the planar (transposing) kernels, checked without a GPU through the library's
test hook sbnet_test_tile_choice: whatever geometry comes in, the tile the host picks must fit what the kernels
assume (registers per thread, LDS, whole coverage of the block plane), and the kernel instances compiled for the
benchmark configurations' shapes must be selected for exactly those shapes."""
import ctypes
import itertools

import pytest

from sbnet_amd import _lib

GATHER_LINES, GATHER_PLANAR, SCATTER_PLANAR = 0, 1, 2
FIELDS = ["threads", "lds", "P", "Pp", "psplit", "Ct", "cchunks", "need", "have", "last", "fixed"]


def choice(kind, R, S, C, num_active, vec=4, H=800, W=800, y_aligned_to=0):
    lib = _lib.load()
    fn = lib.sbnet_test_tile_choice
    fn.restype, fn.argtypes = ctypes.c_int, [ctypes.c_int] * 12 + [ctypes.POINTER(ctypes.c_int32)]
    out = (ctypes.c_int32 * 11)()
    rc = fn(kind, 1, H, W, C, R, S, R, S, num_active, vec, y_aligned_to, out)
    assert rc >= 0
    return dict(zip(FIELDS, out)) if rc else None


def vecs_for(C):
    return [v for v in (4, 2, 1) if C % v == 0]


SIZES = sorted(set(list(range(1, 40)) + [49, 63, 64, 65, 100, 127, 128, 129, 191, 193, 255, 300]))


@pytest.mark.parametrize("kind", [GATHER_PLANAR, SCATTER_PLANAR])
def test_tiles_fit_the_kernels(kind):
    short_tails = 0
    for R, S in itertools.product(SIZES, [1, 2, 3, 5, 16, 27, 31, 63, 65, 127]):
        RS = R * S
        if RS < 4 or RS > 40000:
            continue
        for C in (1, 2, 3, 4, 8, 12, 17, 32, 33, 64, 128, 130):
            for vec in vecs_for(C):
                for num_active in (3, 5000):
                    t = choice(kind, R, S, C, num_active, vec)
                    assert t is not None, (R, S, C, vec)
                    tag = (kind, R, S, C, vec, num_active, t)
                    assert t["threads"] in (64, 128, 256, 512), tag
                    assert t["lds"] == t["Ct"] * t["Pp"] * 4 <= 64 * 1024, tag
                    assert t["Pp"] % 32 == 0 and t["Pp"] >= t["P"], tag
                    assert (t["psplit"] - 1) * t["P"] < RS <= t["psplit"] * t["P"], tag   # the splits tile the plane
                    assert t["last"] == RS - (t["psplit"] - 1) * t["P"] >= 1, tag
                    assert t["Ct"] % vec == 0 and (t["Ct"] // vec) & (t["Ct"] // vec - 1) == 0, tag
                    assert t["cchunks"] * t["Ct"] >= C > (t["cchunks"] - 1) * t["Ct"], tag
                    assert t["need"] <= t["have"], tag   # vectors / slots per thread against the registers that hold them
                    short_tails += t["last"] < 4
    # last splits of fewer than 4 pixels do occur (63x63 with 32 channels ...): the scatter kernel moves those float
    # by float (tests/test_hip_parity.py::test_planar_scatter_short_last_split runs them on the GPU)
    assert short_tails > 0


LINE = 16  # floats per unit of ownership of the line-owning gather: 64 bytes


def test_line_owning_gather_tiles():
    used = 0
    for R, S in itertools.product(SIZES, [5, 16, 18, 27, 31, 63, 65]):
        RS = R * S
        for C in (4, 8, 32, 64, 128, 132):
            for num_active in (3, 300, 5000):
                for align in (0, 16, 64):
                    t = choice(GATHER_LINES, R, S, C, num_active, 4, y_aligned_to=align)
                    if t is None:
                        continue   # whole planes per tile, or a last split shorter than a line: k_gather_planar takes it
                    used += 1
                    tag = (R, S, C, num_active, align, t)
                    assert t["psplit"] >= 2 and (t["psplit"] - 1) * t["P"] < RS <= t["psplit"] * t["P"], tag
                    assert t["last"] >= LINE, tag                     # the last split holds the extension
                    assert t["Pp"] % 32 == 0 and t["Pp"] >= t["P"] + LINE - 1 + 3, tag
                    assert t["lds"] == t["Ct"] * t["Pp"] * 4 <= 64 * 1024, tag
                    assert 4 <= t["have"] <= 8 and t["need"] <= t["have"], tag
    assert used > 100
    # a stack that is not 16-byte aligned cannot be written as whole aligned lines
    assert choice(GATHER_LINES, 27, 27, 128, 312, 4, y_aligned_to=4) is None


def test_fixed_shape_instances_are_selected_for_the_benchmark_shapes_only():
    # 800x800x128, 27x27 blocks: both tile sizes of gather and scatter have an instance
    for M in (58, 156, 312, 1024):
        g, s = choice(GATHER_LINES, 27, 27, 128, M), choice(SCATTER_PLANAR, 27, 27, 128, M)
        assert g["fixed"] == 1 and s["fixed"] == 1, (M, g, s)
    assert choice(GATHER_LINES, 27, 27, 128, 58)["psplit"] == 2 and choice(GATHER_LINES, 27, 27, 128, 312)["psplit"] == 3
    assert choice(SCATTER_PLANAR, 27, 27, 128, 58)["P"] == 184 and choice(SCATTER_PLANAR, 27, 27, 128, 312)["P"] == 124
    assert choice(GATHER_LINES, 18, 18, 64, 75, H=256, W=256)["fixed"] == 1
    assert choice(SCATTER_PLANAR, 16, 16, 64, 75, H=256, W=256)["fixed"] == 1
    # neighbours of those shapes take the run-time-geometry kernels
    for R, S, C in ((27, 27, 64), (27, 26, 128), (26, 27, 128), (27, 27, 132), (18, 18, 128), (16, 16, 32)):
        for kind in (GATHER_LINES, SCATTER_PLANAR):
            t = choice(kind, R, S, C, 312)
            assert t is None or t["fixed"] == 0, (kind, R, S, C, t)
    assert choice(SCATTER_PLANAR, 27, 27, 128, 312, vec=2)["fixed"] == 0
