"""bench.py's host-side pieces that need no GPU: the one-GPU rule, and the rule that `roofline.traffic` is taken from a
counter summary under profiles/ only while the kernel sources are the ones the counters were collected on."""
import os
import subprocess
import sys

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
