"""bench.py's host-side pieces that need no GPU: the one-GPU rule, and the rule that `roofline.traffic` is taken from a
counter summary under profiles/ only while the kernel sources are the ones the counters were collected on."""
import os
import subprocess
import sys

import pytest

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SUMMARY = "gather_lines_scatter_planar_C3_30pct_pmc.txt"


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_kernel_digest_follows_the_sources(tmp_path, monkeypatch):
    d0 = bench.kernel_source_digest()
    assert len(d0) == 64 and d0 == bench.kernel_source_digest()
    csrc = tmp_path / "sbnet_amd" / "csrc"
    csrc.mkdir(parents=True)
    for name in os.listdir(os.path.join(ROOT, "sbnet_amd", "csrc")):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(ROOT, "sbnet_amd", "csrc", name), "rb") as f:
                (csrc / name).write_bytes(f.read())
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    assert bench.kernel_source_digest() == d0
    with open(csrc / "sbnet_launch.h", "ab") as f:
        f.write(b"\n// a comment   and /* another */\n\n")
    assert bench.kernel_source_digest() == d0     # comments and white space are not code
    with open(csrc / "sbnet_launch.h", "ab") as f:
        f.write(b"\nconstexpr int changed = 1;\n")
    assert bench.kernel_source_digest() != d0


def test_counters_of_another_kernel_source_are_not_reported(tmp_path, monkeypatch):
    text = open(os.path.join(ROOT, "profiles", SUMMARY)).read()
    assert "kernel_source_sha256=" in text
    prof = tmp_path / "profiles"
    prof.mkdir()
    monkeypatch.setattr(bench, "kernel_source_digest", lambda: "ab" * 32)
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))

    lines = [ln for ln in text.splitlines() if not ln.startswith("kernel_source_sha256=")]
    (prof / SUMMARY).write_text("\n".join(lines + ["kernel_source_sha256=" + "ab" * 32]) + "\n")
    for op in ("gather", "scatter"):
        got, note = bench.read_measured_traffic(SUMMARY, op)
        # both kernels move at least the stack twice at 30 % density (312 blocks of 27*27*128 floats)
        assert got is not None and got > 2 * 312 * 27 * 27 * 128 * 4 * 0.9, note

    (prof / SUMMARY).write_text("\n".join(lines + ["kernel_source_sha256=" + "cd" * 32]) + "\n")
    got, note = bench.read_measured_traffic(SUMMARY, "gather")
    assert got is None and "stale" in note

    (prof / SUMMARY).write_text("\n".join(lines) + "\n")  # no digest at all: nothing to trust
    assert bench.read_measured_traffic(SUMMARY, "gather")[0] is None
    assert bench.read_measured_traffic("no_such_file.txt", "gather")[0] is None


def test_bench_structs_match_the_cxx_loop():
    """bench.py hands the C++ host loop two structs by pointer; their ctypes mirrors must have the C layout."""
    import ctypes
    so = os.path.join(ROOT, "sbnet_amd", "libsbnet_bench.so")
    lib = ctypes.CDLL(so)
    lib.sbnet_bench_struct_bytes.restype = ctypes.c_size_t
    assert lib.sbnet_bench_struct_bytes(0) == ctypes.sizeof(bench.BenchSet) == 96
    assert lib.sbnet_bench_struct_bytes(1) == ctypes.sizeof(bench.BenchGeom)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["config1", "config2", "config4_small"])
def test_cxx_host_loop_matches_the_oracle(name):
    """The C++ host loop that bench.py times (libsbnet_bench.so) runs the same step as the Python mirror: with a mask
    and a gather (copying scatter at the end), and with a given block list and no gather (in-place atomic add).  Its
    outputs are compared with the CPU oracle, so that the timed step is known to be the op sequence it claims."""
    import numpy as np
    import torch
    from oracle import sbnet_oracle as orc
    from sbnet_amd import _lib, workloads
    lib = _lib.load()
    torch.cuda.set_device(0)
    if name == "config4_small":
        # the overlapping scatter-add configuration's geometry on a small base, block list given
        rng = np.random.default_rng(7)
        cells = np.array([(n, i, j) for n in range(2) for i in range(8) for j in range(8) if rng.random() < 0.3], np.int16)
        wl = workloads.config4()._replace(shape=[2, 64, 64, 32], bcount=[8, 8], indices=cells, name="C4-small")
    else:
        wl = getattr(workloads, name)()
    p = bench.Path(wl, torch, lib, nsets=2)
    if wl.x is None:
        for s in p.sets:
            s["base"].zero_()
    before = [s["base"].clone() for s in p.sets]
    ms = bench.cxx_pipeline(p, 2, 0, 1, device_count=False)["host_count"]   # two steps per call: each set once
    assert ms > 0
    torch.cuda.synchronize()
    M = p.M
    idx = p.idx_host[:M]
    cnt = np.array([M], np.int32)
    for k, s in enumerate(p.sets):
        stack = s["sstack"].cpu().numpy()[:M]
        if wl.x is not None and s["sstack"] is s["stack"]:
            # the loop gathers into a stack of its own (the list's capacity): take the oracle's gather instead
            stack = orc.sparse_gather(wl.x, cnt, idx, wl.bsize, wl.bstride, wl.boffset, transpose=wl.transpose)
        base0 = before[k].cpu().numpy()
        calls = 2 if wl.s_var else 1   # (the loop ran warm-up + timed batch: the in-place op has been applied twice)
        exp = base0
        for _ in range(calls):
            exp = orc.sparse_scatter(stack, cnt, idx, exp, wl.s_bsize, wl.s_bstride, wl.s_boffset, add=wl.s_add,
                                     atomic=wl.s_atomic, transpose=wl.transpose)
        got = (s["base"] if wl.s_var else s["out"]).cpu().numpy()
        np.testing.assert_array_equal(got, exp)
