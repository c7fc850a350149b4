"""The C-ABI boundary on a machine without a GPU: the library loads, exports every symbol that
include/sbnet_amd.h declares, and returns the reference's InvalidArgument conditions before any
device work (reduce_mask.cc:132-138; sparse_gather.cc:164-175, 307-327).  No kernel is launched here."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

from sbnet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
I32x2 = ctypes.c_int32 * 2
I32x3 = ctypes.c_int32 * 3
I64x4 = ctypes.c_int64 * 4
FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: every call below fails validation first


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sbnet_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sbnet_[a-z_]+)\s*\(", text)))


def test_header_declares_what_the_loader_binds():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def _c_kind(ctype):
    """Coarse kind of a C parameter or return type as written in the header."""
    t = " ".join(ctype.replace("const", " ").split())
    if "*" in t:
        return "char*" if t.startswith("char") else "ptr"
    return {"int": "i32", "int32_t": "i32", "unsigned int": "u32", "uint32_t": "u32", "int64_t": "i64",
            "size_t": "size", "float": "f32", "void": "void"}[t]


def _ctypes_kind(t):
    if t is None:
        return "void"
    if t is ctypes.c_char_p:
        return "char*"
    if t is ctypes.c_void_p or isinstance(t, type(ctypes.POINTER(ctypes.c_int))):
        return "ptr"
    return {ctypes.c_int: "i32", ctypes.c_int32: "i32", ctypes.c_uint: "u32", ctypes.c_uint32: "u32",
            ctypes.c_int64: "i64", ctypes.c_size_t: "size", ctypes.c_float: "f32"}[t]


def declared_signatures():
    """name -> (kind of the return type, kinds of the parameters), parsed from the header's declarations."""
    text = open(os.path.join(ROOT, "include", "sbnet_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for ret, name, params in re.findall(r"([A-Za-z_][\w\s\*]*?)\b(sbnet_[a-z_]+)\s*\(([^)]*)\)\s*;", text):
        kinds = []
        for prm in params.split(","):
            prm = " ".join(prm.split())
            if prm in ("void", ""):
                continue
            m = re.match(r"(.*?)(\w+)$", prm)   # type, then the parameter's name
            kinds.append(_c_kind(m.group(1)))
        out[name] = (_c_kind(ret), kinds)
    return out


def test_loader_signatures_match_the_header_declarations():
    """ctypes does not check a prototype: a parameter added on one side only would shift every argument after it.
    Parameter count, order and width class (pointer / 32-bit / 64-bit / size_t / float) of every entry point, as
    the header declares them, against what the loader binds."""
    decl = declared_signatures()
    assert sorted(decl) == sorted(_lib.SIGNATURES)
    for name, (res, args) in _lib.SIGNATURES.items():
        want_res, want_args = decl[name]
        assert _ctypes_kind(res) == want_res, name
        assert [_ctypes_kind(a) for a in args] == want_args, name


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_version_and_status_strings():
    lib = _lib.load()
    assert b"gfx950" in lib.sbnet_version()
    assert b"one-dimensional with shape[0] == 2" in lib.sbnet_status_string(_lib.SBNET_EINVAL_PARAM_SHAPE)
    assert b"Only non-overlapping blocks are supported with add=True, atomic=False" in \
        lib.sbnet_status_string(_lib.SBNET_EINVAL_OVERLAP)
    assert b"rank 4" in lib.sbnet_status_string(_lib.SBNET_EINVAL_RANK)
    assert lib.sbnet_status_string(_lib.SBNET_OK) == b"OK"


def test_size_queries():
    lib = _lib.load()
    assert lib.sbnet_reduce_mask_max_indices(4, I32x2(16, 16), 2) == 1024  # reduce_mask.cc:161
    assert lib.sbnet_reduce_mask_max_indices(4, I32x3(16, 16, 1), 3) == -1
    assert lib.sbnet_reduce_mask_workspace_bytes(4, I32x2(16, 16), 2) >= 1024
    assert lib.sbnet_reduce_mask_workspace_bytes(4, I32x3(1, 1, 1), 3) == 0


def test_scatter_workspace_query():
    lib = _lib.load()
    dims = I64x4(2, 512, 512, 256)
    # the copying scatter built in one pass: one int32 per cell of the block grid, a flag, one int32 per list row
    cells = 2 * 32 * 32 * 4 + 16 + 2000 * 4 + 16
    owner = 2 * 512 * 512 * 4 + 16  # one int32 per pixel: overlapping plain writes in the CPU functor's order
    # blocks that tile (stride == size): no order is needed; the cell map, or the block tables of the atomic-free add
    # (which also serves atomic=1 on tiling blocks) if those are larger
    tables = 2 * 32 * 32 * 4 + 32 + 2000 * 72 * 4
    assert lib.sbnet_sparse_scatter_workspace_bytes(2000, dims, 4, I32x2(16, 16), 2, I32x2(16, 16), 2, I32x2(0, 0),
                                                    2) == max(cells, tables)
    # gaps between the blocks, few of them: the same two candidates
    assert lib.sbnet_sparse_scatter_workspace_bytes(10, dims, 4, I32x2(5, 7), 2, I32x2(16, 16), 2, I32x2(0, 0),
                                                    2) == max(2 * 32 * 32 * 4 + 16 + 10 * 4 + 16,
                                                              2 * 32 * 32 * 4 + 32 + 10 * 72 * 4)
    # 16x16 blocks at stride 8: 2x2 blocks cover a pixel, the atomic-free add applies
    n = lib.sbnet_sparse_scatter_workspace_bytes(2000, dims, 4, I32x2(16, 16), 2, I32x2(8, 8), 2, I32x2(0, 0), 2)
    assert n >= max(2 * 64 * 64 * 4 + 2000 * 4, owner)
    # 16x16 at stride 4: 4x4 blocks cover a pixel: the add runs in 16 passes, which needs the block map only
    # (less than the owner map here)
    n = lib.sbnet_sparse_scatter_workspace_bytes(2000, dims, 4, I32x2(16, 16), 2, I32x2(4, 4), 2, I32x2(0, 0), 2)
    assert n == owner
    # 16x16 at stride 3: 6x6 blocks cover a pixel, beyond both atomic-free adds: the owner map only
    assert lib.sbnet_sparse_scatter_workspace_bytes(2000, dims, 4, I32x2(16, 16), 2, I32x2(3, 3), 2, I32x2(0, 0),
                                                    2) == owner
    # an image of 2^30 floats or more is beyond the one-pass copy; the owner map still applies to it
    big = I64x4(1, 32768, 32768, 1)
    assert lib.sbnet_sparse_scatter_workspace_bytes(2000, big, 4, I32x2(16, 16), 2, I32x2(3, 3), 2, I32x2(0, 0),
                                                    2) == 32768 * 32768 * 4 + 16
    assert lib.sbnet_sparse_scatter_workspace_bytes(2000, dims, 3, I32x2(16, 16), 2, I32x2(8, 8), 2, I32x2(0, 0),
                                                    2) == 0


def test_reduce_mask_param_shape_errors():
    lib = _lib.load()
    ok = I32x2(2, 2)
    bad = I32x3(2, 2, 2)
    for pos in range(4):
        ptrs = [ok, ok, ok, ok]
        lens = [2, 2, 2, 2]
        ptrs[pos], lens[pos] = bad, 3
        rc = lib.sbnet_reduce_mask(FAKE, 1, 4, 4, ptrs[0], lens[0], ptrs[1], lens[1], ptrs[2], lens[2], ptrs[3],
                                   lens[3], 0.5, 0, FAKE, None, FAKE, None, 0, None)
        assert rc == _lib.SBNET_EINVAL_PARAM_SHAPE
    # arguments the reference never checks but that would fault a kernel
    rc = lib.sbnet_reduce_mask(None, 1, 4, 4, ok, 2, ok, 2, ok, 2, ok, 2, 0.5, 0, FAKE, None, FAKE, None, 0, None)
    assert rc == _lib.SBNET_EINVAL_ARG
    rc = lib.sbnet_reduce_mask(FAKE, 1, 4, 4, ok, 2, ok, 2, ok, 2, ok, 2, 0.5, 0, FAKE, None, None, None, 0, None)
    assert rc == _lib.SBNET_EINVAL_ARG  # no count destination at all
    rc = lib.sbnet_reduce_mask(FAKE, 1, 4, 4, I32x2(40000, 2), 2, ok, 2, ok, 2, ok, 2, 0.5, 0, FAKE, None, FAKE,
                               None, 0, None)
    assert rc == _lib.SBNET_EINVAL_ARG  # bh would not fit the int16 index triple
    rc = lib.sbnet_reduce_mask(FAKE, 1, 4, 4, ok, 2, ok, 2, ok, 2, ok, 2, 0.5, 0, FAKE, None, FAKE, FAKE, 8, None)
    assert rc == _lib.SBNET_EINVAL_ARG  # workspace too small
    rc = lib.sbnet_reduce_mask_functor(FAKE, 1, 4, 4, 0.5, 0, 0, 2, 2, 2, 2, 2, 2, 2, 2, FAKE, FAKE, 0, None, 0,
                                       None)
    assert rc == _lib.SBNET_EINVAL_ARG  # numBins must be 1 (reduce_mask.cc:69)


def test_gather_errors():
    lib = _lib.load()
    ok = I32x2(2, 2)
    dims = I64x4(1, 4, 4, 1)
    assert lib.sbnet_sparse_gather(FAKE, dims, 3, 1, FAKE, ok, 2, ok, 2, ok, 2, 0, FAKE, None) == \
        _lib.SBNET_EINVAL_RANK
    assert lib.sbnet_sparse_gather(FAKE, dims, 4, 1, FAKE, ok, 2, I32x3(1, 1, 1), 3, ok, 2, 0, FAKE, None) == \
        _lib.SBNET_EINVAL_PARAM_SHAPE
    # rank is checked before the parameter vectors (sparse_gather.cc:164 then :169-175)
    assert lib.sbnet_sparse_gather(FAKE, dims, 5, 1, FAKE, ok, 1, ok, 2, ok, 2, 0, FAKE, None) == \
        _lib.SBNET_EINVAL_RANK
    assert lib.sbnet_sparse_gather(FAKE, dims, 4, -1, FAKE, ok, 2, ok, 2, ok, 2, 0, FAKE, None) == \
        _lib.SBNET_EINVAL_ARG
    assert lib.sbnet_sparse_gather(FAKE, dims, 4, 1, None, ok, 2, ok, 2, ok, 2, 0, FAKE, None) == \
        _lib.SBNET_EINVAL_ARG
    # zero active blocks is a no-op, not an error
    assert lib.sbnet_sparse_gather(FAKE, dims, 4, 0, None, ok, 2, ok, 2, ok, 2, 0, None, None) == _lib.SBNET_OK


@pytest.mark.parametrize("var", [False, True])
def test_scatter_errors(var):
    lib = _lib.load()
    dims = I64x4(1, 4, 4, 1)
    size, overlap, ok = I32x2(2, 2), I32x2(1, 2), I32x2(2, 2)

    def call(rank, bstride, blen, add, atomic):
        if var:
            return lib.sbnet_sparse_scatter_var(FAKE, 1, FAKE, FAKE, dims, rank, size, 2, bstride, blen, ok, 2, add,
                                                atomic, 0, None, 0, None)
        return lib.sbnet_sparse_scatter(FAKE, 1, FAKE, FAKE, dims, rank, size, 2, bstride, blen, ok, 2, add, atomic,
                                        0, ctypes.c_void_p(0x100000), None, 0, None)

    assert call(4, overlap, 2, 1, 0) == _lib.SBNET_EINVAL_OVERLAP      # sparse_gather.cc:322-326
    assert call(3, overlap, 2, 1, 0) == _lib.SBNET_EINVAL_OVERLAP      # tested before the rank
    assert call(3, overlap, 2, 1, 1) == _lib.SBNET_EINVAL_RANK         # sparse_gather.cc:327
    assert call(3, overlap, 2, 0, 0) == _lib.SBNET_EINVAL_RANK
    assert call(4, I32x3(2, 2, 2), 3, 0, 0) == _lib.SBNET_EINVAL_PARAM_SHAPE  # sparse_gather.cc:307-313


def test_scatter_rejects_aliasing_output():
    lib = _lib.load()
    dims = I64x4(1, 4, 4, 1)
    ok = I32x2(2, 2)
    rc = lib.sbnet_sparse_scatter(FAKE, 1, FAKE, FAKE, dims, 4, ok, 2, ok, 2, ok, 2, 0, 0, 0,
                                  ctypes.c_void_p(0x1000 + 16), None, 0, None)
    assert rc == _lib.SBNET_EINVAL_ARG


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs a host C++ compiler")
def test_reference_functor_header_compiles_links_and_reports_errors():
    """include/sbnet_reference_functors.hpp gives the reference's functor templates (reduce_mask.h:23-44,
    sparse_gather.h:23-76) their GPU specialisations on top of the C ABI.  tests/cxx/functor_shim_check.cpp uses it
    as a build of the reference would and calls every functor with arguments the library rejects before any
    device work."""
    subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "tests", "cxx"), "_build/functor_shim_check"], check=True,
                   capture_output=True, text=True)
    exe = os.path.join(ROOT, "tests", "cxx", "_build", "functor_shim_check")
    out = subprocess.run([exe], check=True, capture_output=True, text=True)
    assert "functor shim ok" in out.stdout


def test_python_mirror_checks_sizes_before_any_launch():
    """The kernels trust the count, the list and the stack shapes: the Python mirror refuses what would make them
    read or write past an allocation (the reference's ops do not check these, sparse_gather.cc:190-192, 332)."""
    import torch
    from sbnet_amd import ops

    idx = torch.zeros((5, 3), dtype=torch.int16)
    ops._check_count(0, idx)
    ops._check_count(5, idx)
    for bad in (-1, 6):
        with pytest.raises(ops.InvalidArgument, match="outside the block list"):
            ops._check_count(bad, idx)
    ops._check_stack(torch.zeros((5, 3, 4, 8)), 5, 8, 3, 4, False, "x")
    ops._check_stack(torch.zeros((7, 8, 3, 4)), 5, 8, 3, 4, True, "x")
    for shape, transpose in (((4, 3, 4, 8), False),      # fewer blocks than the count
                             ((5, 8, 3, 4), False),      # planar stack given as NHWC
                             ((5, 3, 4, 8), True),       # and the other way round
                             ((5, 3, 4, 7), False),      # channel count of another tensor
                             ((5, 3, 4), False)):        # not rank 4
        with pytest.raises(ops.InvalidArgument, match="block stack of shape"):
            ops._check_stack(torch.zeros(shape), 5, 8, 3, 4, transpose, "x")


@pytest.mark.gpu
def test_scratch_provider_keeps_outgrown_buffers_until_shutdown():
    """sbnet_scratch_acquire hands one grow-only buffer per stream to callers without an allocator.  A pointer it
    has handed out stays valid when a later, larger request on the same stream replaces the buffer (another thread
    may have asked in between): the outgrown buffer is kept until sbnet_shutdown.  release_workspaces() drops the
    Python mirror's buffers as well, and the ops work again afterwards."""
    import numpy as np
    import torch
    import sbnet_amd
    lib = _lib.load()
    assert lib.sbnet_shutdown() == 0
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    small = lib.sbnet_scratch_acquire(1 << 20, stream)
    assert small and lib.sbnet_scratch_acquire(4096, stream) == small     # fits: the same buffer
    src = torch.arange(1 << 18, dtype=torch.float32, device="cuda:0")
    large = lib.sbnet_scratch_acquire(8 << 20, stream)                    # grows: a new buffer
    assert large and large != small
    # the first pointer is still device memory the caller may use (work queued on it may not have run yet)
    assert lib.sbnet_copy_tensor(small, src.data_ptr(), 1 << 18, stream) == 0
    back = torch.empty_like(src)
    assert lib.sbnet_copy_tensor(back.data_ptr(), small, 1 << 18, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(back, src)
    assert lib.sbnet_scratch_acquire(2 << 20, stream) == large
    free_before = torch.cuda.mem_get_info()[0]
    sbnet_amd.release_workspaces()                                         # sbnet_shutdown inside
    assert torch.cuda.mem_get_info()[0] >= free_before + (8 << 20)
    mask = torch.ones((1, 8, 8, 1), device="cuda:0")
    r = sbnet_amd.reduce_mask(mask, [2, 2], [4, 4], [4, 4], [0, 0], tol=0.5)
    assert int(r.bin_counts[0]) == 4
    assert np.array_equal(r.active_block_indices.cpu().numpy()[:4], [[0, 0, 0], [0, 0, 1], [0, 1, 0], [0, 1, 1]])


def test_python_mirror_fails_loudly_without_library(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsbnet_amd.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()
