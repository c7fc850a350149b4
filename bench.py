#!/usr/bin/env python3
"""Benchmark of the reduce_mask -> sparse_gather -> sparse_scatter path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--density 0.30] [--all-configs] [--only C5] [--no-cpu]

A step is one pass of the path over the LiDAR-BEV-shaped workload (x = [1,800,800,128] fp32,
27x27 blocks, stride 25, offset -1, max pooling, tol 0.5, `--density` of the 1024 blocks active):
reduce_mask, sparse_gather with the fused transpose, and sparse_scatter_var in place (add=False, same
geometry).  Inputs are resident in HBM before the timed region; three independent buffer sets (more
than 1 GB in total) are rotated so the 256 MB Infinity Cache cannot serve one step's data to the next.
All calls go through the C ABI of libsbnet_amd.so with ctypes; PyTorch only owns the device buffers
and the stream.

The step is timed several ways (`pipeline` in the output): with the reference's host-visible count
(reduce_mask returns once the count has reached the host, which sizes the other launches), with the count left on the
device (the `_device_count` entry points, three calls per step), each driven from a C++ host loop
(libsbnet_bench.so, built from sbnet_amd/csrc/sbnet_bench_loop.cpp) and from Python, and with the three launches captured
in a HIP graph and replayed.  One JSON line goes to stdout.  `value` is algorithmic bytes per step /
wall time per step under the reference's contract (host-visible count) from the C++ loop; the others are reported
beside it.  Each is the median of 15 batches of `--steps` steps.  `ops`
holds per-op device times (HIP events around batches of back-to-back launches on the launch stream) at
`--density`, `ops_by_density` the same at 5 %, 15 % and 30 %,
`roofline` the dominant kernel (the slower of gather and scatter) against the 8 TB/s HBM peak, `cpu_baseline`
the single-threaded CPU oracle (the reference's CPU functors restated; the reference builds them
without OpenMP) on the same workload on this machine's host cores.  `ops_nhwc` times the same gather and
scatter with transpose=False (the reference's default layout), `configs` holds the other four benchmark
configurations (end to end and per op), `reference_layer_sizes` the three shapes on which the reference's own
test times gather + scatter (sbnet_ops/tests/test_sparse_blocks.py:440-443).

Every per-op entry carries two byte counts.  `algorithmic_bytes` is the reference's data flow (the table below).
`moved_bytes` is what this implementation has to move for the same result: an ordered overlapping write stores
every covered pixel once, not once per covering block; the owner-computes overlapping add reads and writes every
covered pixel once and reads only the in-image part of the stack; the copying scatter is built in one pass (the
base is read where it is needed and the output written once) instead of copy-then-scatter.  Fractions of the
8 TB/s peak are given for both; the second is the one that says how close the kernel is to the memory system.

Algorithmic bytes (B = bsize[0]*bsize[1]*C*4 per block, B_in its in-image part, M active blocks):
  gather            M*(B_in + B) + 6*M      read x once per block element, write the stack
  scatter add=False M*(B + B_in) + 6*M      read the stack, write the base
  scatter add=True  M*(B + 2*B_in) + 6*M    read the stack, read-modify-write the base
  reduce_mask       N*H*W*4 + 6*M + 4       every mask pixel once
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--density", type=float, default=0.30)
    ap.add_argument("--all-configs", action="store_true")
    ap.add_argument("--only", default=None, metavar="NAME",
                    help="time one configuration only (C1, C2, C3@5%%, C3@15%%, C3@30%%, C4, C5, or `layers` for the reference's "
                         "layer shapes) and print its row to "
                         "stdout instead of the benchmark line: for profiling the other configurations' kernels")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline (profiling runs)")
    ap.add_argument("--ops-only", action="store_true",
                    help="per-op tables only (ops_by_density), no pipeline timing: a kernel trace of this run holds "
                         "exactly the launches the per-op times and the roofline come from")
    ap.add_argument("--kernel-digest", action="store_true",
                    help="print the digest of the kernel sources (the `kernel_source_sha256=` line a counter summary "
                         "under profiles/ carries) and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run the library's plain copy kernel on 256 MiB, 10 times: a kernel of known traffic "
                         "against which profiler byte counters are scaled")
    return ap.parse_args()


I2 = ctypes.c_int32 * 2
I64x4 = ctypes.c_int64 * 4


def in_image_bytes(idx, bsize, bstride, boffset, H, W, C):
    """Sum over blocks of the in-image part of the block, in bytes."""
    h0 = boffset[0] + idx[:, 1].astype(np.int64) * bstride[0]
    w0 = boffset[1] + idx[:, 2].astype(np.int64) * bstride[1]
    rows = np.clip(np.minimum(h0 + bsize[0], H) - np.maximum(h0, 0), 0, None)
    cols = np.clip(np.minimum(w0 + bsize[1], W) - np.maximum(w0, 0), 0, None)
    return int((rows * cols).sum()) * C * 4


def covered_pixels(idx, bsize, bstride, boffset, N, H, W):
    """Number of distinct in-image pixels that the blocks of the list cover."""
    cov = np.zeros((N, H, W), bool)
    for n, bh, bw in np.asarray(idx, np.int64):
        if 0 <= n < N:
            h0, w0 = boffset[0] + bh * bstride[0], boffset[1] + bw * bstride[1]
            cov[n, max(h0, 0):max(h0 + bsize[0], 0), max(w0, 0):max(w0 + bsize[1], 0)] = True
    return int(cov.sum())


class Path:
    """Pre-allocated device buffers and raw C-ABI calls for one workload, `nsets` rotating copies."""

    def __init__(self, wl, torch, lib, nsets=3, stack_fill=None):
        self.wl, self.torch, self.lib = wl, torch, lib
        dev = "cuda:0"
        N, H, W, C = wl.shape
        self.N, self.H, self.W, self.C = N, H, W, C
        self.dims = I64x4(N, H, W, C)
        self.bc, self.bs, self.bst, self.bo = I2(*wl.bcount), I2(*wl.bsize), I2(*wl.bstride), I2(*wl.boffset)
        self.sbs, self.sbst, self.sbo = I2(*wl.s_bsize), I2(*wl.s_bstride), I2(*wl.s_boffset)
        self.maxidx = N * wl.bcount[0] * wl.bcount[1]
        self.nws = lib.sbnet_reduce_mask_workspace_bytes(N, self.bc, 2)
        self.use_scatter_ws = True
        self.host_count = np.zeros(1, np.int32)
        self.hc_ptr = self.host_count.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.sets = []
        if wl.indices is not None:
            idx_host = np.ascontiguousarray(wl.indices, np.int16)
            self.M = len(idx_host)
        else:
            # the block list comes from the library's own reduce_mask (untimed): it sizes the buffers
            mask_d = torch.from_numpy(wl.mask).to(dev)
            idx_d = torch.zeros((self.maxidx, 3), dtype=torch.int16, device=dev)
            ws_d = torch.empty(max(self.nws, 16), dtype=torch.uint8, device=dev)
            self.check(lib.sbnet_reduce_mask(mask_d.data_ptr(), N, H, W, self.bc, 2, self.bs, 2, self.bst, 2, self.bo, 2,
                                             wl.tol, int(wl.avgpool), idx_d.data_ptr(), self.hc_ptr, None,
                                             ws_d.data_ptr(), self.nws, self.stream))
            torch.cuda.synchronize()
            self.M = int(self.host_count[0])
            idx_host = idx_d[:self.M].cpu().numpy()
            del mask_d, idx_d, ws_d
        self.idx_host = idx_host
        R, S = wl.bsize
        sR, sS = wl.s_bsize
        for i in range(nsets):
            s = {}
            if wl.mask is not None:
                s["mask"] = torch.from_numpy(wl.mask).to(dev)
                s["idx"] = torch.zeros((self.maxidx, 3), dtype=torch.int16, device=dev)
                s["idx"][:self.M] = torch.from_numpy(idx_host).to(dev)
            else:
                s["mask"] = None
                s["idx"] = torch.from_numpy(idx_host).to(dev)
            s["ws"] = torch.empty(max(self.nws, 16), dtype=torch.uint8, device=dev)
            # every scatter is given the scratch the library asks for: overlapping adds then run without atomics,
            # overlapping plain writes land in the CPU functor's order, the copying op is built in one pass
            # (sized for the whole list, which the device-count entry points take as their capacity)
            nsw = lib.sbnet_sparse_scatter_workspace_bytes(max(self.M, self.maxidx), self.dims, 4, self.sbs, 2, self.sbst,
                                                           2, self.sbo, 2)
            s["sws"] = torch.empty(nsw, dtype=torch.uint8, device=dev) if nsw else None
            s["dcount"] = torch.zeros(1, dtype=torch.int32, device=dev)
            if wl.x is not None:
                s["x"] = torch.from_numpy(wl.x).to(dev)
                s["stack"] = torch.empty((self.M, C, R, S) if wl.transpose else (self.M, R, S, C),
                                         dtype=torch.float32, device=dev)
            else:
                s["x"] = None
            shape = (self.M, C, sR, sS) if wl.transpose else (self.M, sR, sS, C)
            if (sR, sS) == (R, S) and wl.x is not None:
                s["sstack"] = s["stack"]
            else:
                g = torch.Generator(device=dev).manual_seed(4000 + i)
                s["sstack"] = torch.rand(shape, generator=g, device=dev) * 2.0 - 1.0
            s["base"] = torch.zeros((N, H, W, C), dtype=torch.float32, device=dev) if wl.x is None or not wl.s_var \
                else s["x"]
            if not wl.s_var:
                s["out"] = torch.empty((N, H, W, C), dtype=torch.float32, device=dev)
            self.sets.append(s)
        torch.cuda.synchronize()
        B = R * S * C * 4
        sB = sR * sS * C * 4
        bin_g = in_image_bytes(idx_host, wl.bsize, wl.bstride, wl.boffset, H, W, C)
        bin_s = in_image_bytes(idx_host, wl.s_bsize, wl.s_bstride, wl.s_boffset, H, W, C)
        M = self.M
        full = N * H * W * C * 4
        self.bytes = {
            "reduce_mask": N * H * W * 4 + 6 * M + 4,
            "gather": bin_g + M * B + 6 * M,
            "scatter": M * sB + (2 if wl.s_add else 1) * bin_s + 6 * M + (0 if wl.s_var else 2 * full),
        }
        # what this implementation has to move (see the module docstring)
        cov = covered_pixels(idx_host, wl.s_bsize, wl.s_bstride, wl.s_boffset, N, H, W) * C * 4
        if not wl.s_var:
            sc = M * sB + (full if wl.s_add else full - cov) + full + 6 * M
        elif not wl.s_add:
            sc = M * sB + cov + 6 * M
        elif wl.s_atomic:
            sc = bin_s + 2 * cov + 6 * M
        else:
            sc = M * sB + 2 * bin_s + 6 * M
        self.moved = {"reduce_mask": self.bytes["reduce_mask"], "gather": self.bytes["gather"], "scatter": sc}
        # the gradient of the gather: as the reference composes it (zeros_like(x) written, then the atomic scatter-add
        # reads the stack and reads and writes every covered element once per covering block); and what has to move
        # (the stack read once, the tensor written once)
        self.bytes["gather_backward"] = full + M * B + 2 * bin_g + 6 * M
        self.moved["gather_backward"] = full + M * B + 6 * M

    def check(self, rc):
        if rc != 0:
            raise RuntimeError("sbnet call failed: %s (hip %d)" % (self.lib.sbnet_status_string(rc).decode(),
                                                                    self.lib.sbnet_last_hip_error()))

    def reduce(self, i, sync=True):
        s, wl = self.sets[i], self.wl
        self.check(self.lib.sbnet_reduce_mask(s["mask"].data_ptr(), self.N, self.H, self.W, self.bc, 2, self.bs, 2,
                                              self.bst, 2, self.bo, 2, wl.tol, int(wl.avgpool), s["idx"].data_ptr(),
                                              self.hc_ptr if sync else None, s["dcount"].data_ptr(),
                                              s["ws"].data_ptr(), self.nws, self.stream))
        return int(self.host_count[0]) if sync else self.M

    def gather(self, i, M):
        s, wl = self.sets[i], self.wl
        self.check(self.lib.sbnet_sparse_gather(s["x"].data_ptr(), self.dims, 4, M, s["idx"].data_ptr(), self.bs, 2,
                                                self.bst, 2, self.bo, 2, int(wl.transpose), s["stack"].data_ptr(),
                                                self.stream))

    def scatter(self, i, M):
        s, wl = self.sets[i], self.wl
        ws = s["sws"] if self.use_scatter_ws else None
        wp, wn = (ws.data_ptr(), ws.numel()) if ws is not None else (None, 0)
        if wl.s_var:
            self.check(self.lib.sbnet_sparse_scatter_var(s["sstack"].data_ptr(), M, s["idx"].data_ptr(),
                                                         s["base"].data_ptr(), self.dims, 4, self.sbs, 2, self.sbst, 2,
                                                         self.sbo, 2, int(wl.s_add), int(wl.s_atomic),
                                                         int(wl.transpose), wp, wn, self.stream))
        else:
            self.check(self.lib.sbnet_sparse_scatter(s["sstack"].data_ptr(), M, s["idx"].data_ptr(),
                                                     s["base"].data_ptr(), self.dims, 4, self.sbs, 2, self.sbst, 2,
                                                     self.sbo, 2, int(wl.s_add), int(wl.s_atomic), int(wl.transpose),
                                                     s["out"].data_ptr(), wp, wn, self.stream))

    def step_device_count(self, i):
        """The same three ops with the count left on the device (entry points with the _device_count suffix):
        launches are sized for the whole list (max_active = N*bcount_h*bcount_w) and nothing waits for the host."""
        s, wl = self.sets[i], self.wl
        if "stack_cap" not in s:
            R, S = wl.bsize
            s["stack_cap"] = self.torch.empty((self.maxidx, self.C, R, S) if wl.transpose else
                                              (self.maxidx, R, S, self.C), dtype=self.torch.float32, device="cuda:0")
        self.reduce(i, sync=False)
        self.check(self.lib.sbnet_sparse_gather_device_count(
            s["x"].data_ptr(), self.dims, 4, s["dcount"].data_ptr(), self.maxidx, s["idx"].data_ptr(), self.bs, 2,
            self.bst, 2, self.bo, 2, int(wl.transpose), s["stack_cap"].data_ptr(), self.stream))
        ws = s["sws"]
        self.check(self.lib.sbnet_sparse_scatter_var_device_count(
            s["stack_cap"].data_ptr(), s["dcount"].data_ptr(), self.maxidx, s["idx"].data_ptr(), s["base"].data_ptr(),
            self.dims, 4, self.sbs, 2, self.sbst, 2, self.sbo, 2, int(wl.s_add), int(wl.s_atomic), int(wl.transpose),
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, self.stream))

    def step(self, i):
        M = self.reduce(i) if self.wl.mask is not None else self.M
        if self.wl.x is not None:
            self.gather(i, M)
        self.scatter(i, M)
        return M

    def time_op(self, fn, batches=7, reps=24):
        """Median device time per launch: HIP events around `reps` back-to-back launches on the stream
        the kernels run on (torch's current stream), rotating over the buffer sets.  Two launches go ahead
        of the first event so that the host is ahead of the device when the timed region starts; on an idle
        stream the first event completes at once and the region would include the host's launch latency."""
        torch = self.torch
        n = len(self.sets)
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        out = []
        for b in range(batches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            fn((b * reps - 2) % n)
            fn((b * reps - 1) % n)
            e0.record()
            for r in range(reps):
                fn((b * reps + r) % n)
            e1.record()
            e1.synchronize()
            out.append(e0.elapsed_time(e1) * 1e3 / reps)
        return statistics.median(out)

    def gather_grad(self, i, M):
        """The gradient of the gather with respect to x (sbnet_sparse_gather_grad): the stack scattered and summed
        onto zeros; written into the set's `grad` tensor."""
        s, wl = self.sets[i], self.wl
        if "grad" not in s:
            s["grad"] = self.torch.empty((self.N, self.H, self.W, self.C), dtype=self.torch.float32, device="cuda:0")
            n = self.lib.sbnet_sparse_scatter_workspace_bytes(max(self.M, self.maxidx), self.dims, 4, self.bs, 2, self.bst, 2,
                                                              self.bo, 2)
            s["gws"] = self.torch.empty(max(n, 16), dtype=self.torch.uint8, device="cuda:0")
        self.check(self.lib.sbnet_sparse_gather_grad(s["stack"].data_ptr(), M, s["idx"].data_ptr(), s["grad"].data_ptr(),
                                                     self.dims, 4, self.bs, 2, self.bst, 2, self.bo, 2, int(wl.transpose),
                                                     s["gws"].data_ptr(), s["gws"].numel(), self.stream))

    def op_table(self, with_gather_grad=False):
        ops = {}
        if self.wl.mask is not None:
            ops["reduce_mask"] = self.time_op(lambda i: self.reduce(i, sync=False))
        if self.wl.x is not None:
            ops["gather"] = self.time_op(lambda i: self.gather(i, self.M))
        ops["scatter"] = self.time_op(lambda i: self.scatter(i, self.M))
        if with_gather_grad and self.wl.x is not None:
            ops["gather_backward"] = self.time_op(lambda i: self.gather_grad(i, self.M))
            for s in self.sets:
                s.pop("grad", None)
                s.pop("gws", None)
        table = {}
        for k, us in ops.items():
            gbs, mgbs = self.bytes[k] / us * 1e-3, self.moved[k] / us * 1e-3
            table[k] = {"us": round(us, 2), "algorithmic_bytes": self.bytes[k], "moved_bytes": self.moved[k],
                        "GBps": round(gbs, 1), "frac_of_8TBps": round(gbs / HBM_PEAK_GBS, 4),
                        "moved_GBps": round(mgbs, 1), "moved_frac_of_8TBps": round(mgbs / HBM_PEAK_GBS, 4)}
        return table


class BenchSet(ctypes.Structure):   # struct sbnet_bench_set of sbnet_amd/csrc/sbnet_bench_loop.cpp
    _fields_ = [("mask", ctypes.c_void_p), ("x", ctypes.c_void_p), ("base", ctypes.c_void_p),
                ("stack", ctypes.c_void_p), ("idx", ctypes.c_void_p), ("count_dev", ctypes.c_void_p),
                ("reduce_ws", ctypes.c_void_p), ("reduce_ws_bytes", ctypes.c_size_t),
                ("scatter_ws", ctypes.c_void_p), ("scatter_ws_bytes", ctypes.c_size_t),
                ("scatter_stack", ctypes.c_void_p), ("out", ctypes.c_void_p)]


class BenchGeom(ctypes.Structure):  # struct sbnet_bench_geom
    _fields_ = [("N", ctypes.c_int), ("H", ctypes.c_int), ("W", ctypes.c_int), ("C", ctypes.c_int),
                ("bcount", I2), ("bsize", I2), ("bstride", I2), ("boffset", I2),
                ("s_bsize", I2), ("s_bstride", I2), ("s_boffset", I2),
                ("tol", ctypes.c_float), ("avgpool", ctypes.c_int), ("transpose", ctypes.c_int),
                ("add", ctypes.c_int), ("atomic", ctypes.c_int), ("max_active", ctypes.c_int32),
                ("fixed_count", ctypes.c_int32)]


def cxx_pipeline(path, steps, warmup, batches, device_count=True):
    """The step driven by a C++ host loop over the same C ABI (libsbnet_bench.so): ms per step of the median batch,
    for the reference's contract (mode 0, count handed to the host) and, for the in-place pipeline, with the count
    on the device (mode 1).  Workloads without a mask or without x skip those ops; the copying op writes `out`."""
    so = os.path.join(ROOT, "sbnet_amd", "libsbnet_bench.so")
    if not os.path.exists(so):
        raise RuntimeError("%s is not built; run `make -C sbnet_amd/csrc`" % so)
    lib_so = ctypes.CDLL(so)
    lib_so.sbnet_bench_struct_bytes.restype = ctypes.c_size_t
    if (lib_so.sbnet_bench_struct_bytes(0), lib_so.sbnet_bench_struct_bytes(1)) != \
            (ctypes.sizeof(BenchSet), ctypes.sizeof(BenchGeom)):
        raise RuntimeError("BenchSet / BenchGeom do not match the structs of sbnet_bench_loop.cpp; rebuild %s" % so)
    loop = lib_so.sbnet_bench_pipeline
    loop.restype = ctypes.c_int
    loop.argtypes = [ctypes.POINTER(BenchSet), ctypes.c_int, ctypes.POINTER(BenchGeom), ctypes.c_int, ctypes.c_int,
                     ctypes.c_void_p, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int32)]
    wl, torch = path.wl, path.torch
    R, S = wl.bsize
    ptr = lambda t: t.data_ptr() if t is not None else None
    # the gathered stack at the list's capacity (the device-count launches cover all of it) where a gather runs
    caps = [torch.empty((path.maxidx, path.C, R, S) if wl.transpose else (path.maxidx, R, S, path.C),
                        dtype=torch.float32, device="cuda:0") if s["x"] is not None else None for s in path.sets]
    sets = (BenchSet * len(path.sets))()
    for k, s in enumerate(path.sets):
        sws = s["sws"]
        # the scatter reads the gathered stack where both ops share a block size, else a stack of its own size
        sstack = caps[k] if s.get("stack") is not None and s["sstack"] is s["stack"] else s["sstack"]
        sets[k] = BenchSet(ptr(s["mask"]), ptr(s["x"]), s["base"].data_ptr(), ptr(caps[k]),
                           s["idx"].data_ptr(), s["dcount"].data_ptr(), s["ws"].data_ptr(), path.nws,
                           ptr(sws), sws.numel() if sws is not None else 0, sstack.data_ptr(), ptr(s.get("out")))
    g = BenchGeom(path.N, path.H, path.W, path.C, I2(*wl.bcount), I2(*wl.bsize), I2(*wl.bstride), I2(*wl.boffset),
                  I2(*wl.s_bsize), I2(*wl.s_bstride), I2(*wl.s_boffset), wl.tol, int(wl.avgpool), int(wl.transpose),
                  int(wl.s_add), int(wl.s_atomic), path.maxidx, path.M)
    out = {}
    sec, cnt = ctypes.c_double(0.0), ctypes.c_int32(0)
    for mode, name in ((0, "host_count"), (1, "device_count"))[:2 if device_count else 1]:
        path.check(loop(sets, len(path.sets), ctypes.byref(g), max(warmup, len(path.sets)), mode, path.stream,
                        ctypes.byref(sec), ctypes.byref(cnt)))
        per = []
        for _ in range(batches):
            path.check(loop(sets, len(path.sets), ctypes.byref(g), steps, mode, path.stream, ctypes.byref(sec),
                            ctypes.byref(cnt)))
            assert cnt.value == path.M, "active block count changed between runs"
            per.append(sec.value / steps * 1e3)
        out[name] = statistics.median(per)
    del caps
    torch.cuda.empty_cache()
    return out


def cpu_baseline(wl, M, idx_host, nbytes, budget_s=12.0):
    """Times the CPU oracle's gather + scatter (single thread: the reference's Makefile has no -fopenmp)
    on the same workload, repeating until about `budget_s` seconds have been spent."""
    from oracle import sbnet_oracle as orc
    lib = orc.lib()
    x = wl.x
    N, H, W, C = wl.shape
    R, S = wl.bsize
    stack = np.empty((M, C, R, S) if wl.transpose else (M, R, S, C), np.float32)
    base = x.copy()
    f32p = ctypes.POINTER(ctypes.c_float)
    i16p = ctypes.POINTER(ctypes.c_int16)
    idx = np.ascontiguousarray(idx_host, np.int16)

    def run(omp):
        g = lib.oracle_sparse_gather_omp if omp else lib.oracle_sparse_gather
        sc = lib.oracle_sparse_scatter_omp if omp else lib.oracle_sparse_scatter
        t0 = time.perf_counter()
        g(x.ctypes.data_as(f32p), N, H, W, C, stack.ctypes.data_as(f32p), wl.boffset[0], wl.boffset[1], R, S,
          wl.bstride[0], wl.bstride[1], M, idx.ctypes.data_as(i16p), int(wl.transpose))
        sc(stack.ctypes.data_as(f32p), N, H, W, C, base.ctypes.data_as(f32p), wl.s_boffset[0], wl.s_boffset[1],
           wl.s_bsize[0], wl.s_bsize[1], wl.s_bstride[0], wl.s_bstride[1], M, idx.ctypes.data_as(i16p), int(wl.s_add),
           int(wl.transpose), 0)
        return time.perf_counter() - t0

    run(False)
    times, spent = [], 0.0
    while spent < budget_s * 0.7 and len(times) < 400:
        t = run(False)
        times.append(t)
        spent += t
    t1 = statistics.median(times)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    omp_threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    run(True)
    times_omp, spent = [], 0.0
    while spent < budget_s * 0.3 and len(times_omp) < 400:
        t = run(True)
        times_omp.append(t)
        spent += t
    tm = statistics.median(times_omp)
    sample = "%s gather(transpose)+scatter_var, full workload (M=%d blocks), median of %d runs" % (wl.name, M, len(times))
    return ({"value": round(nbytes / t1 * 1e-9, 3), "unit": "GB/s", "cores": 1, "kind": "port", "sample": sample,
             "ms_per_pass": round(t1 * 1e3, 2)},
            {"value": round(nbytes / tm * 1e-9, 3), "unit": "GB/s", "cores": omp_threads, "kind": "port",
             "sample": sample.replace("median of %d" % len(times), "median of %d" % len(times_omp)) + ", OpenMP over blocks",
             "ms_per_pass": round(tm * 1e3, 2)})


def copy_rate(torch, lib, batches=7, reps=24):
    """What a flat copy reaches on this box: the library's copy kernel (sbnet_copy_tensor: nontemporal 16-byte loads
    and stores, 16 KB per workgroup) on 256 MiB, three rotating buffer pairs, timed like the ops (HIP events around
    batches of back-to-back launches on the launch stream).  The block movers are copies with index arithmetic, so
    this is the practical ceiling their rates are to be read against, beside the 8 TB/s of the data sheet."""
    n = 64 * 1024 * 1024  # floats
    src = [torch.ones(n, device="cuda:0") for _ in range(3)]
    dst = [torch.empty(n, device="cuda:0") for _ in range(3)]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def fn(i):
        rc = lib.sbnet_copy_tensor(dst[i % 3].data_ptr(), src[i % 3].data_ptr(), n, st)
        assert rc == 0

    for i in range(3):
        fn(i)
    torch.cuda.synchronize()
    per = []
    for b in range(batches):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn(0)
        fn(1)
        e0.record()
        for r in range(reps):
            fn(b * reps + r)
        e1.record()
        e1.synchronize()
        per.append(e0.elapsed_time(e1) * 1e3 / reps)
    us = statistics.median(per)
    del src, dst
    torch.cuda.empty_cache()
    gbps = 2 * n * 4 / us * 1e-3
    return {"kernel": "k_copy_v4 (sbnet_copy_tensor), 256 MiB read + 256 MiB written per launch", "us": round(us, 2),
            "GBps": round(gbps, 1), "frac_of_8TBps": round(gbps / HBM_PEAK_GBS, 4)}


def kernel_source_digest():
    """sha256 over the code of the device sources the library is built from (csrc/*.hip and csrc/*.h, by name,
    comments and white space left out): the counters under profiles/ belong to one state of it."""
    import glob
    import hashlib
    import re
    d = os.path.join(ROOT, "sbnet_amd", "csrc")
    h = hashlib.sha256()
    for p in sorted(glob.glob(os.path.join(d, "*.hip")) + glob.glob(os.path.join(d, "*.h"))):
        with open(p, "r") as f:
            text = f.read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
        text = re.sub(r"//[^\n]*", " ", text)      # (no string literal in these files holds "//")
        h.update(os.path.basename(p).encode() + b"\0" + " ".join(text.split()).encode() + b"\0")
    return h.hexdigest()


def read_measured_traffic(name, op):
    """HBM bytes per launch of `op` ("gather" or "scatter") measured with rocprofv3 --pmc, if a summary under
    profiles/ records them as lines `<op>_fetch_bytes_per_launch=<int>` and `<op>_write_bytes_per_launch=<int>`.
    Returns (bytes, note).  The summary names the kernel source it was measured on (`kernel_source_sha256=`); when
    the source has changed since, the counters no longer describe these kernels and the bytes are None."""
    p = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(p):
        return None, "no counter summary under profiles/"
    vals, digest = {}, None
    for line in open(p):
        line = line.strip()
        if line.startswith("kernel_source_sha256="):
            digest = line.split("=", 1)[1].split()[0]
        for key in ("%s_fetch_bytes_per_launch" % op, "%s_write_bytes_per_launch" % op):
            if line.startswith(key + "="):
                vals[key] = int(float(line.split("=", 1)[1].split()[0]))
    if len(vals) != 2:
        return None, "profiles/%s holds no counters for the %s" % (name, op)
    if digest != kernel_source_digest():
        return None, ("profiles/%s was measured on another state of the kernel sources: its counters are stale "
                      "until its commands are run again" % name)
    return sum(vals.values()), ("profiles/%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the copy kernel, on "
                                "this kernel source; not re-measured by this run)" % name)


def main():
    args = parse()
    if args.kernel_digest:
        print(kernel_source_digest())
        return
    if args.gpus != 1:
        print("bench.py: this path is measured on one GPU only (one MI355X per box); --gpus %d is not supported. "
              "The path shards by image (n) with no exchange between GPUs." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from sbnet_amd import _lib, workloads
    lib = _lib.load()
    torch.cuda.set_device(0)

    if args.copy_calibration:
        n = 64 * 1024 * 1024  # floats: 256 MiB read + 256 MiB written per launch
        src = [torch.ones(n, device="cuda:0") for _ in range(3)]
        dst = [torch.empty(n, device="cuda:0") for _ in range(3)]
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for i in range(10):
            rc = lib.sbnet_copy_tensor(dst[i % 3].data_ptr(), src[i % 3].data_ptr(), n, st)
            assert rc == 0
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if args.only == "layers":
        print(json.dumps(layer_rows(torch, lib, workloads)))
        return
    if args.only:
        if args.only not in CONFIGS:
            print("bench.py: --only takes one of %s" % ", ".join(CONFIGS), file=sys.stderr)
            sys.exit(2)
        print(json.dumps(config_row(args.only, torch, lib, workloads)))
        return

    # per-op device times at the three densities the configuration sweeps; the buffers of the density the
    # pipeline is timed on (--density) are kept for the step timings below
    densities = sorted(set([0.05, 0.15, 0.30, args.density]))
    ops_by_density = {}
    path = None
    for d in densities:
        p = Path(workloads.config3(d), torch, lib, nsets=3)
        table = p.op_table(with_gather_grad=(d == args.density))
        table["M"] = p.M
        ops_by_density["%d%%" % round(d * 100)] = table
        if d == args.density:
            path, wl, ops = p, p.wl, table
        else:
            del p
            torch.cuda.empty_cache()
    if args.ops_only:
        print(json.dumps({"ops_by_density": ops_by_density}))
        return
    nsets = len(path.sets)
    step_bytes = path.bytes["reduce_mask"] + path.bytes["gather"] + path.bytes["scatter"]
    BATCHES = 15

    def timed(step_fn):
        """W untimed steps, then BATCHES batches of exactly K steps, each between two device synchronisations;
        ms per step of the median batch (K steps of 0.1 ms are too short a sample to quote one batch)."""
        for i in range(max(args.warmup, nsets)):
            step_fn(i % nsets)
        torch.cuda.synchronize()
        per = []
        for b in range(BATCHES):
            t0 = time.perf_counter()
            for i in range(args.steps):
                step_fn((b * args.steps + i) % nsets)
            torch.cuda.synchronize()
            per.append((time.perf_counter() - t0) / args.steps * 1e3)
        return statistics.median(per)

    def variant(ms, note):
        return {"ms_per_step": round(ms, 4), "GBps": round(step_bytes / (ms * 1e-3) * 1e-9, 1), "note": note}

    # (1) the reference's contract: reduce_mask hands the count to the host, which sizes the other two launches
    counts = []
    host_ms = timed(lambda i: counts.append(path.step(i)))
    assert counts[-1] == path.M, "active block count changed between runs"

    # (2) the count stays on the device: launches sized for max_active blocks, nothing waits for the host
    dc_ms = timed(path.step_device_count)
    dc_counts = [int(s["dcount"].cpu()[0]) for s in path.sets]
    assert dc_counts == [path.M] * nsets, "device-resident count differs from the host-visible one"

    # (3) the same three launches captured once per buffer set into a HIP graph and replayed
    eager_stream = path.stream
    graphs = []
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        path.stream = ctypes.c_void_p(side.cuda_stream)
        for i in range(nsets):
            path.step_device_count(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in range(nsets):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            path.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            path.step_device_count(i)
        graphs.append(g)
    path.stream = eager_stream
    for s in path.sets:
        s["dcount"].zero_()
    graph_ms = timed(lambda i: graphs[i].replay())
    dc_counts = [int(s["dcount"].cpu()[0]) for s in path.sets]
    assert dc_counts == [path.M] * nsets, "graph replay produced a different count"
    del graphs
    for s in path.sets:
        s.pop("stack_cap", None)
    torch.cuda.empty_cache()

    # (4) the first two again from a C++ host loop: what a caller written in the reference's host language sees
    cxx = cxx_pipeline(path, args.steps, args.warmup, BATCHES)

    # `value`: the pipeline under the reference's contract (reduce_mask returns with the count on the host, gather
    # and scatter are sized from it), driven from C++.  The other variants are reported beside it.
    ms_per_step = cxx["host_count"]
    value = step_bytes / (ms_per_step * 1e-3) * 1e-9

    # the dominant kernel: whichever of the two block movers takes longer per launch, in the launch shape `value`
    # uses (grids sized from the host count, which is what the per-op table times)
    dom = "gather" if ops["gather"]["us"] >= ops["scatter"]["us"] else "scatter"
    g = ops[dom]
    kernel_names = {"gather": "planar gather of sparse_gather(transpose=True): k_gather_lines",
                    "scatter": "planar scatter of sparse_scatter_var(add=False, transpose=True): k_scatter_planar"}
    traffic_file = "gather_lines_scatter_planar_C3_30pct_pmc.txt"
    if round(args.density * 100) == 30:
        traffic, traffic_note = read_measured_traffic(traffic_file, dom)
    else:
        traffic, traffic_note = None, "counters were collected at 30 % density only"
    roofline = {"bound": "hbm", "kernel": kernel_names[dom],
                "achieved": g["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(g["GBps"] / HBM_PEAK_GBS, 4), "us_per_launch": g["us"],
                "algorithmic_bytes_per_launch": g["algorithmic_bytes"], "moved_bytes_per_launch": g["moved_bytes"],
                "traffic": traffic, "traffic_source": traffic_note}
    if traffic:
        # the same launch time against the bytes the profiler counted between L2 and the fabric
        roofline["traffic_GBps"] = round(traffic / g["us"] * 1e-3, 1)
    # a flat copy on the same box, timed the same way: what a copy-shaped kernel can reach here
    flat = copy_rate(torch, lib)
    roofline["flat_copy"] = flat
    roofline["frac_of_flat_copy"] = round(g["GBps"] / flat["GBps"], 4)
    out = {
        "metric": "achieved HBM GB/s over reduce_mask+sparse_gather+sparse_scatter_var (algorithmic bytes / wall time per step); us/op and % of HBM peak under ops, ops_by_density and roofline",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "C3 LiDAR-BEV x=[1,800,800,128] fp32, bsize 27 bstride 25 boffset -1, max-pool tol 0.5, "
                               "%d%% of 1024 blocks active (M=%d), gather transpose=True, scatter_var add=False in place"
                               % (round(args.density * 100), path.M),
                   "buffer_sets": nsets, "bytes_per_step": step_bytes,
                   "timing": "median of %d batches of %d steps, each batch between two device synchronisations"
                             % (BATCHES, args.steps)},
        "ops": ops, "ops_by_density": ops_by_density, "roofline": roofline,
        "pipeline": {
            "host_count_reference_contract_cxx": variant(cxx["host_count"],
                                                         "value: reduce_mask returns with the count on the host (the "
                                                         "reference's HostMemory output; stored into pinned memory by "
                                                         "the kernel and polled), gather and scatter sized from it; "
                                                         "three C-ABI calls per step from a C++ loop "
                                                         "(sbnet_amd/csrc/sbnet_bench_loop.cpp)"),
            "device_count_cxx": variant(cxx["device_count"], "count read on the device (entry points only this library "
                                                             "has), launches sized for max_active=%d blocks, same "
                                                             "C++ loop" % path.maxidx),
            "host_count_reference_contract": variant(host_ms, "the reference's contract with the three calls made "
                                                              "from Python through ctypes"),
            "device_count_eager": variant(dc_ms, "count read on the device, three calls per step from Python"),
            "device_count_graph": variant(graph_ms, "count read on the device, reduce_mask + gather + scatter_var "
                                                    "captured in one HIP graph per buffer set, one replay per step"),
        },
    }
    if not args.no_cpu:
        nb = path.bytes["gather"] + path.bytes["scatter"]
        one, omp = cpu_baseline(wl, path.M, path.idx_host, nb)
        out["cpu_baseline"] = one
        out["cpu_baseline_openmp"] = omp
        gpu_gs = nb / ((ops["gather"]["us"] + ops["scatter"]["us"]) * 1e-6) * 1e-9
        out["gather_plus_scatter_GBps"] = round(gpu_gs, 1)
    del path
    torch.cuda.empty_cache()

    # the same two ops in the reference's default layout (transpose=False), same workload
    p = Path(workloads.config3(args.density)._replace(transpose=False), torch, lib, nsets=3)
    t = p.op_table()
    out["ops_nhwc"] = {"gather": t["gather"], "scatter": t["scatter"], "M": p.M,
                       "note": "sparse_gather / sparse_scatter_var with transpose=False (NHWC block stack), %s" % p.wl.name}
    del p
    torch.cuda.empty_cache()

    # the other benchmark configurations, each end to end (host-visible count) and per op
    out["configs"] = {name: config_row(name, torch, lib, workloads) for name in ("C1", "C2", "C4", "C5")}

    out["reference_layer_sizes"] = layer_rows(torch, lib, workloads)
    print(json.dumps(out))
    sys.stdout.flush()

    if args.all_configs:
        for name in CONFIGS:
            if name.startswith("C3"):
                print(json.dumps(config_row(name, torch, lib, workloads)), file=sys.stderr)


CONFIGS = ["C1", "C2", "C3@5%", "C3@15%", "C3@30%", "C4", "C5"]


def layer_rows(torch, lib, workloads):
    """The shapes the reference's own test times its gather + scatter on (timed region: both ops)."""
    layers = {}
    for size in workloads.REFERENCE_LAYER_SIZES:
        for transpose in (False, True):
            p = Path(workloads.reference_layer(size, transpose), torch, lib, nsets=3)
            t = p.op_table()
            layers["%dx%dx%d %s" % (size + ("transpose" if transpose else "nhwc",))] = {
                "M": p.M, "gather": t["gather"], "scatter": t["scatter"],
                "gather_plus_scatter_us": round(t["gather"]["us"] + t["scatter"]["us"], 2)}
            del p
            torch.cuda.empty_cache()
    return {"note": "benchmarkLayerSizes of the reference's test (18x18 blocks at stride 18, offset (-1,-2), every block "
                    "active): sparse_gather, then the copying sparse_scatter(add=False); the reference times both ops "
                    "together with its in-graph timers",
            "rows": layers}


def config_row(name, torch, lib, workloads):
    """End-to-end time (host-visible count) and per-op device times of one configuration."""
    gens = {"C1": (workloads.config1, {}), "C2": (workloads.config2, {}), "C3@5%": (workloads.config3, {"density": 0.05}),
            "C3@15%": (workloads.config3, {"density": 0.15}), "C3@30%": (workloads.config3, {"density": 0.30}),
            "C4": (workloads.config4, {}), "C5": (workloads.config5, {})}
    gen, kw = gens[name]
    p = Path(gen(**kw), torch, lib, nsets=2 if name == "C4" else 3)
    n = len(p.sets)
    for i in range(5):
        p.step(i % n)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    K = 50
    for i in range(K):
        p.step(i % n)
    torch.cuda.synchronize()
    e2e = (time.perf_counter() - t0) / K * 1e6
    wl = p.wl
    cxx = cxx_pipeline(p, K, 5, 5, device_count=False)["host_count"] * 1e3
    row = {"config": name, "M": p.M, "end_to_end_us": round(e2e, 1), "end_to_end_cxx_us": round(cxx, 1),
           "ops": p.op_table(),
           "workload": "x=%s bsize %s bstride %s boffset %s %s-pool tol %g; gather transpose=%s; %s add=%s atomic=%s "
                       "bsize %s bstride %s boffset %s" % (
                           wl.shape, wl.bsize, wl.bstride, wl.boffset, "avg" if wl.avgpool else "max", wl.tol,
                           wl.transpose, "sparse_scatter_var" if wl.s_var else "sparse_scatter", wl.s_add, wl.s_atomic,
                           wl.s_bsize, wl.s_bstride, wl.s_boffset)}
    del p
    torch.cuda.empty_cache()
    return row


if __name__ == "__main__":
    main()
