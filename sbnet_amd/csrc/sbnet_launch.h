// Host-side launch interface between the C ABI (sbnet_capi.cpp) and the gfx950 kernels
// (sbnet_reduce_mask.hip, sbnet_gather.hip, sbnet_scatter.hip).  Everything here takes already-validated arguments.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace sbnet {

// Block geometry shared by the three ops.  Block (n, bh, bw) covers
// x[n, oh + U*bh : oh + U*bh + R, ow + V*bw : ow + V*bw + S, :].
struct Geom {
    int N, H, W, C;
    int R, S;    // block size  (bsize)
    int U, V;    // block stride (bstride)
    int oh, ow;  // block offset (boffset)
    // Optional: device-resident length of the block list.  When set, the kernels treat numActive as the
    // capacity of the list and skip rows at or beyond *countDev, so no host round trip is needed between
    // reduce_mask and its consumers.
    const int32_t* countDev;
    // Tests only: never launch a fixed-shape kernel instance, so that the run-time-geometry kernels are covered
    // for the shapes that have instances too.
    int forceGeneric;
};

enum ScatterMode { SCATTER_ASSIGN = 0, SCATTER_ADD = 1, SCATTER_ATOMIC = 2 };

// reduce_mask scratch: one flag byte per sparsity block, one int32 count per pooling workgroup, one int32 for
// the total when the caller gives no device count.  Its contents before a
// call do not matter.  reduce_mask_count_slot: where the total goes when the caller gives no device count.
size_t reduce_mask_workspace_bytes(int64_t totalBlocks);
int32_t* reduce_mask_count_slot(void* workspace, int64_t totalBlocks);

// hostSignal (optional): device-visible address of an 8-byte word in pinned host memory; the kernel that knows
// the count stores (hostSeq << 32 | count) there, so a host that polls the word needs no copy and no stream
// synchronisation to learn the count.
hipError_t launch_reduce_mask(const float* mask, const Geom& g, int bCntH, int bCntW, float tol,
                              bool avgPool, bool fixupZero, int16_t* activeBlockIndices,
                              int32_t* binCountDevice, void* workspace, hipStream_t stream,
                              unsigned long long* hostSignal = nullptr, uint32_t hostSeq = 0);

// Device address of the library's own scratch array on the current device (STATIC_SCRATCH_BYTES bytes, 256-byte
// aligned): no allocation, looked up once per device.  Every call on a GPU shares that GPU's array.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)2 << 20;
hipError_t static_scratch(void** ptr);

// Test hook: see tile_choice in sbnet_gather.hip.
int tile_choice(int kind, const Geom& g, int numActive, int vec, int yAlignedTo, int32_t* out);

hipError_t launch_gather(const float* x, float* y, const int16_t* idx, int numActive,
                         const Geom& g, bool transpose, hipStream_t stream);

hipError_t launch_scatter(const float* x, float* y, const int16_t* idx, int numActive,
                          const Geom& g, bool transpose, ScatterMode mode, hipStream_t stream);

// Scatter-add on overlapping blocks without atomics (NHWC stack only): bit-identical to the sequential CPU
// order.  Needs scratch of scatter_pull_workspace_bytes(); `done` is false when the method does not apply
// (no or too little scratch, more than 2x2 blocks covering a pixel) and nothing was launched.
size_t scatter_pull_workspace_bytes(const Geom& g, int numActive);
hipError_t launch_scatter_pull(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                               void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done);

// Scatter-add on overlapping blocks in ceil(R/U)*ceil(S/V) passes of plain load-add-store, one residue class of
// block positions per pass (either stack layout, up to 16 passes): reproducible, within rounding of the
// sequential order.  Needs scratch of scatter_color_workspace_bytes(); `done` as above.
size_t scatter_color_workspace_bytes(const Geom& g, int numActive);
// ontoZeros: y is uninitialised and the result is zeros plus the blocks; the zeros are written by the call, and only
// where no block covers a pixel when at most 2x2 blocks do (the passes then store a pixel's first value instead of
// adding to it).
hipError_t launch_scatter_colored(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                  bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream,
                                  bool& done, bool ontoZeros = false);
hipError_t launch_zero(float* y, size_t count, hipStream_t stream);
// The same result (zeros plus the sum of overlapping blocks) in one pass over the stack: every covered pixel is
// written once, by the block listed last over it, as the sum in list order of the blocks that cover it; at most 2x2
// blocks over a pixel, scratch of scatter_color_workspace_bytes().
hipError_t launch_scatter_onto_zeros(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                     bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done);

// Plain writes ("=") of overlapping blocks in the order of the sequential CPU functor: on a pixel that several
// blocks cover, the block listed last wins (sparse_gather.cc:105-129), for either stack layout and for lists that
// name a block twice.  Needs scratch of scatter_owner_workspace_bytes() (one int32 per pixel; 0 when the blocks do
// not overlap and no order is needed); `done` is false when that is missing and nothing was launched.
size_t scatter_owner_workspace_bytes(const Geom& g, int numActive);
hipError_t launch_scatter_owned(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done);

// y = copy of ybase with the blocks written ("=") or added ("+=", non-overlapping) on top, moving every byte once.
// Blocks that do not overlap: an inverse map (cell of the block grid -> list position) in the scratch, then one
// streaming kernel over y that reads ybase where the result needs it, the stack where a block covers the pixel,
// and writes y once (planar stacks of geometries the kernel does not stage: a pass that copies the uncovered
// pixels, then the scatter kernels, which read ybase where they add).  Overlapping plain writes: the owner map of
// the ordered scatter as coverage record, a copy of the uncovered pixels, then the ordered scatter.  Needs scratch
// of scatter_cover_workspace_bytes() / scatter_owner_workspace_bytes(); `done` is false when the method does not
// apply (no scratch, atomic mode, too little coverage to pay for the extra launches) and nothing was launched:
// the caller then copies ybase and scatters in place.
size_t scatter_cover_workspace_bytes(const Geom& g, int numActive);
hipError_t launch_scatter_over_base(const float* x, const float* ybase, float* y, const int16_t* idx, int numActive,
                                    const Geom& g, bool transpose, ScatterMode mode, void* workspace,
                                    size_t workspaceBytes, hipStream_t stream, bool& done);

hipError_t launch_copy(float* dst, const float* src, size_t count, hipStream_t stream);

}  // namespace sbnet
