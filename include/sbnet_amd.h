/*
 * sbnet_amd.h -- C ABI of libsbnet_amd.so: the three Sparse Blocks Network custom ops
 * (reduce_mask, sparse_gather, sparse_scatter / sparse_scatter_var) as hand-written HIP kernels
 * for gfx950 (MI355X).
 *
 * The entry points replace the reference's TensorFlow op kernels and the functors below them
 * (paths relative to the reference checkout, sbnet_tensorflow/sbnet_ops/).  Two levels exist,
 * as in the reference:
 *
 *   op level       what OpKernel::Compute does: parameter validation, the host-visible count,
 *                  the zero-count fix-up, copy-before-scatter.   Names: sbnet_<op>.
 *   functor level  what Functor<GPUDevice,float>::operator() does: launch only, reference
 *                  argument order.                               Names: sbnet_<op>_functor.
 *
 * Conventions
 *   - Only float32 tensors, NHWC, C-contiguous.  Block indices are int16 triples (n, bh, bw)
 *     (reduce_mask.cc:109, sparse_gather.cc:53).
 *   - The caller owns every buffer.  Pointers are device pointers unless a parameter says "host".
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  All work is
 *     enqueued on it; only sbnet_reduce_mask with a host count pointer waits for it.
 *   - The dynamic_b* parameters are host int32 arrays with an explicit length so that the
 *     reference's "should be one-dimensional with shape[0] == 2" check can be mirrored.
 *   - Every function returns an sbnet_status.  No function ever calls exit(); the reference
 *     prints and exits on a device error (op_utils.h:27-35), this library returns SBNET_EHIP.
 *   - Re-entrant.  What the library keeps between calls: a thread-local last-error slot, one pinned
 *     count word per thread and device (sbnet_reduce_mask with a host count), and the buffers of
 *     sbnet_scratch_acquire for callers that use it; sbnet_shutdown frees the last two.
 */
#ifndef SBNET_AMD_H
#define SBNET_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sbnet_status {
    SBNET_OK = 0,
    /* dynamic_b<count,size,stride,offset> not length 2
       (reduce_mask.cc:132-138, sparse_gather.cc:169-175, 307-313). */
    SBNET_EINVAL_PARAM_SHAPE = 1,
    /* x / ybase not rank 4 (sparse_gather.cc:164, 327). */
    SBNET_EINVAL_RANK = 2,
    /* add && !atomic with bstride < bsize (sparse_gather.cc:322-326). */
    SBNET_EINVAL_OVERLAP = 3,
    /* Anything the reference does not check but that would make a kernel read or write out of
       bounds: NULL pointers, non-positive sizes, dimensions beyond the int16 index range,
       a workspace that is too small, y aliasing ybase in the copying scatter. */
    SBNET_EINVAL_ARG = 4,
    /* A HIP runtime call failed; sbnet_last_hip_error() has the hipError_t. */
    SBNET_EHIP = 5,
    /* sbnet_reduce_mask_static: the problem needs more scratch than the library's own array holds. */
    SBNET_ETOOBIG = 6
} sbnet_status;

/* Human-readable text for a status; the InvalidArgument texts are the reference's. */
const char* sbnet_status_string(int status);
/* hipError_t of the last SBNET_EHIP on the calling thread (0 if none). */
int sbnet_last_hip_error(void);
const char* sbnet_version(void);

/* ------------------------------------------------------------------------------------------
 * reduce_mask
 * ---------------------------------------------------------------------------------------- */

/* Rows of active_block_indices the caller must allocate: N * bcount[0] * bcount[1]
   (reduce_mask.cc:161).  Returns -1 on bad arguments. */
int64_t sbnet_reduce_mask_max_indices(int N, const int32_t* bcount, int bcount_len);

/* Bytes of device scratch sbnet_reduce_mask / _functor need for this problem size. */
size_t sbnet_reduce_mask_workspace_bytes(int N, const int32_t* bcount, int bcount_len);

/*
 * Op level: replaces ReduceMaskOp<GPUDevice,float>::Compute (reduce_mask.cc:123-221).
 *
 *   mask                  device fp32 [N,H,W,1]
 *   bcount/bsize/bstride/boffset   host int32[2] each (len must be 2)
 *   tol, avgpool          op attributes (reduce_mask.cc:102-103).  max mode: active if any
 *                         in-range pixel > tol.  avg mode: active if sum(in-range)/(bsize[0]*
 *                         bsize[1]) > tol, with the sum taken in the CPU functor's row-major
 *                         order (reduce_mask.cc:78-88), so results are identical to the
 *                         reference's CPU path for any mask, not only binary ones.
 *   active_block_indices  device int16 [max_indices, 3].  Unlike the reference's GPU kernel
 *                         (arbitrary order, reduce_mask.cu.h:141-154) rows are written in the
 *                         CPU functor's lexicographic (n, bh, bw) order.  Rows past the count
 *                         are left untouched.
 *   bin_counts_host       host int32[1] or NULL.  Non-NULL keeps the reference's HostMemory
 *                         contract (reduce_mask.cc:198-220): the call returns once the count is
 *                         in *bin_counts_host.  The kernel that knows the count stores it into a
 *                         word of pinned host memory (one per calling thread and device, allocated
 *                         on first use) which the call polls, so there is no device-to-host copy
 *                         and no stream synchronisation; active_block_indices is complete in stream
 *                         order, like any other output.  Where that word cannot be had, the count
 *                         is copied and the stream synchronised as the reference does.  Not
 *                         available while `stream` is being captured into a graph (SBNET_EHIP).
 *                         NULL: nothing reaches the host, the call is asynchronous.
 *   bin_counts_device     device int32[1] or NULL; receives the same count.  At least one of
 *                         the two count pointers must be non-NULL.
 *   A mask with no active block reports count 1 and writes the triple (0,0,0)
 *   (reduce_mask.cc:206-218); the fix-up happens on the device, without a host round trip.
 *   workspace             device scratch of sbnet_reduce_mask_workspace_bytes() bytes, 16-byte
 *                         aligned, or NULL to let the call allocate and free its own
 *                         (slower, and it synchronises the stream; refused with SBNET_EHIP /
 *                         hipErrorStreamCaptureUnsupported, before anything is allocated or enqueued,
 *                         while `stream` is being captured).
 */
int sbnet_reduce_mask(const float* mask, int N, int H, int W,
                      const int32_t* bcount, int bcount_len,
                      const int32_t* bsize, int bsize_len,
                      const int32_t* bstride, int bstride_len,
                      const int32_t* boffset, int boffset_len,
                      float tol, int avgpool,
                      int16_t* active_block_indices,
                      int32_t* bin_counts_host, int32_t* bin_counts_device,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * sbnet_reduce_mask for callers that cannot allocate and have no workspace to bring: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  The
 * scratch is an array inside the library's code object (2 MiB per GPU, held until the process ends); the call
 * allocates nothing, on the device or the host, and frees nothing.  For the same reason the count goes to
 * bin_counts_device only (required): the host-visible count of sbnet_reduce_mask needs a word of pinned host
 * memory.  Everything else (arguments, checks, order of the list, zero-count fix-up, asynchronous on `stream`)
 * is sbnet_reduce_mask's.
 *   Limit: N * bcount[0] * bcount[1] <= sbnet_reduce_mask_static_max_indices() (about 400 000 blocks);
 *   beyond that the call returns SBNET_ETOOBIG and launches nothing.
 *   Every call on a GPU uses that GPU's one array: calls that may run at the same time on one GPU (different
 *   streams, different threads) race on it and must be serialised by the caller; calls on one stream are.
 *   Nothing in the array has to be cleared between calls (every byte of it that a call reads has been
 *   written by that call), so a smaller problem may follow a larger one.
 *   The first call on a device looks the array's device address up (hipGetSymbolAddress, once per device, under
 *   a mutex): make that call outside stream capture; every later call does no HIP call but its kernel launches
 *   and may be captured.
 */
int sbnet_reduce_mask_static(const float* mask, int N, int H, int W,
                             const int32_t* bcount, int bcount_len,
                             const int32_t* bsize, int bsize_len,
                             const int32_t* bstride, int bstride_len,
                             const int32_t* boffset, int boffset_len,
                             float tol, int avgpool,
                             int16_t* active_block_indices, int32_t* bin_counts_device, void* stream);
int64_t sbnet_reduce_mask_static_max_indices(void);

/*
 * Functor level: replaces ReduceMaskFunctor<GPUDevice,float>::operator()
 * (reduce_mask.h:23-44, reduce_mask.cu:39-89).  Same argument order; numBins must be 1 as the
 * reference asserts (reduce_mask.cc:69), binSize is ignored.  binCounts is a device int32[1]
 * and receives the raw count (0 is possible: the fix-up belongs to the op level).
 */
int sbnet_reduce_mask_functor(const float* mask, int N, int H, int W, float threshold,
                              int bOffsH0, int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW,
                              int bCntH, int bCntW, unsigned int numBins, unsigned int binSize,
                              int16_t* activeBlockIndices, int32_t* binCounts, int avgPool,
                              void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * sparse_gather
 * ---------------------------------------------------------------------------------------- */

/*
 * Op level: replaces SparseGatherOp<GPUDevice,float>::Compute (sparse_gather.cc:160-218).
 *
 *   x, x_dims, x_rank     device fp32 NHWC and its shape; rank must be 4
 *   num_active            bin_counts[0], which the reference reads on the host
 *                         (sparse_gather.cc:190-192)
 *   active_block_indices  device int16 [>= num_active, 3]
 *   transpose             0: y is [num_active, bsize[0], bsize[1], C]
 *                         1: y is [num_active, C, bsize[0], bsize[1]]  (sparse_gather.cc:197-204)
 *   y                     device fp32, caller-allocated with that shape
 *   Pixels outside the image read as 0 (sparse_gather.cc:80-82).
 */
int sbnet_sparse_gather(const float* x, const int64_t* x_dims, int x_rank,
                        int32_t num_active, const int16_t* active_block_indices,
                        const int32_t* bsize, int bsize_len,
                        const int32_t* bstride, int bstride_len,
                        const int32_t* boffset, int boffset_len,
                        int transpose, float* y, void* stream);

/* Functor level: replaces SparseGatherFunctor<GPUDevice,float>::operator()
   (sparse_gather.h:23-42, sparse_gather.cu:62-154). */
int sbnet_sparse_gather_functor(const float* x, int N, int H, int W, int C, float* y,
                                int bOffsH0, int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW,
                                int numActive, const int16_t* activeBlockIndices, int transpose,
                                void* stream);

/* Gradient of sparse_gather with respect to x.  The reference registers it as a composition of its own ops,
   sparse_scatter(grad, bin_counts, indices, zeros_like(x), ..., add=True, atomic=True, transpose)
   (sparse_conv_lib.py:80-107, the same text in sbnet_ops/tests/test_sparse_blocks.py:36-62); this entry point computes
   that tensor without materialising the zeros first:
     dx = 0 everywhere, plus every block of dy at the block's place; where blocks overlap their values are summed.
   dy is the block stack of the forward op's output layout ([num_active, R, S, C], or [num_active, C, R, S] with
   transpose=1), dx a caller-allocated tensor of x's shape whose contents on entry do not matter.  With `workspace`
   (sbnet_sparse_scatter_workspace_bytes() bytes for the same geometry) and at most 2x2 blocks over a pixel, zeros
   are written only to the pixels that no block covers, and one pass over the stack writes every other pixel once:
   the block listed last over a pixel fetches the other blocks' values of it and stores 0 + their sum in list order
   + its own.  No atomics: the result is the sequential CPU functor's (sparse_gather.cc:105-129), bit for bit, also
   for real-valued data and signed zeros, and the same on every call.  A list that names a block twice falls back
   to hardware atomics onto zeros; deeper overlaps take ceil(R/U)*ceil(S/V) passes of mutually non-overlapping
   blocks (reproducible, equal to the composition up to fp32 reassociation); without workspace dx is cleared and
   the atomic scatter-add runs on it.  Checks and status codes as sbnet_sparse_scatter_var. */
int sbnet_sparse_gather_grad(const float* dy, int32_t num_active, const int16_t* active_block_indices, float* dx,
                             const int64_t* x_dims, int x_rank,
                             const int32_t* bsize, int bsize_len,
                             const int32_t* bstride, int bstride_len,
                             const int32_t* boffset, int boffset_len,
                             int transpose, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * sparse_scatter / sparse_scatter_var
 * ---------------------------------------------------------------------------------------- */

/* Bytes of scratch that let an overlapping atomic scatter-add run without atomics, that give overlapping plain
   writes the CPU functor's order, and that let sparse_scatter build its output in one pass instead of copying
   ybase first (see workspace below); 0 when none of these applies to this geometry. */
size_t sbnet_sparse_scatter_workspace_bytes(int32_t num_active, const int64_t* ybase_dims, int ybase_rank,
                                            const int32_t* bsize, int bsize_len,
                                            const int32_t* bstride, int bstride_len,
                                            const int32_t* boffset, int boffset_len);

/*
 * Op level: replaces SparseScatterOp<GPUDevice,float,false>::Compute (sparse_gather.cc:286-357,
 * registered as "SparseScatter", sparse_gather.cc:256-268): y = copy(ybase), then the blocks of
 * x are written (add=0), added (add=1) or atomically added (add=1, atomic=1) on top of y.
 * Unlike the reference (sparse_gather.cu:268-276) the copy does not synchronise the stream.
 *
 *   x           device fp32 block stack: [num_active, bsize[0], bsize[1], C], or
 *               [num_active, C, bsize[0], bsize[1]] when transpose=1 (sparse_gather.cc:117-120)
 *   ybase       device fp32 [N,H,W,C]; ybase_dims/ybase_rank give its shape, rank must be 4
 *   y           device fp32, same shape, must not overlap ybase
 *   Pixels of a block that fall outside the image are dropped (sparse_gather.cc:121).
 *   add=1, atomic=0 requires bstride >= bsize on both axes (sparse_gather.cc:322-326).
 *   add=0 with overlapping blocks (bstride < bsize): the reference's CPU functor walks the list front to
 *   back, so the block listed last wins on a pixel that several blocks cover (sparse_gather.cc:105-129).
 *   This library writes exactly that, for both stack layouts and for lists that name a block twice: without
 *   scratch when at most 2x2 blocks cover a pixel (bsize <= 2*bstride) and the list has at most 2048 blocks
 *   (planar stack, transpose=1) or 192 blocks (NHWC stack): the kernel that moves a block compares it with
 *   the rows listed after it; otherwise given scratch (below).  Where neither holds, as in the reference's
 *   GPU path, which block wins is unspecified unless the overlapping values are equal.
 *   workspace   optional device scratch (4-byte aligned) of sbnet_sparse_scatter_workspace_bytes() bytes,
 *               or NULL.  Three uses.
 *               (0) add=0 and bstride < bsize, where the kernel cannot order the blocks itself (long lists,
 *               more than 2x2 blocks over a pixel): every block writes only the pixels that no
 *               block listed later covers: the CPU functor's result, no pixel written twice.  Which pixels
 *               those are comes from one small extra launch that compares the blocks of the list pairwise (at
 *               most 2x2 blocks over a pixel and at most 4096 blocks; in-place op), or else from an owner map
 *               (one int32 per pixel: the last listed block that covers it) built by two extra launches.
 *               (1) sbnet_sparse_scatter with atomic=0 and blocks that do not overlap (bstride >= bsize): y is
 *               built in one pass over its bytes instead of "copy ybase, scatter on top".  One or two small
 *               launches put an inverse map (block position -> list position) into the scratch; one streaming kernel
 *               then walks y in row order, reads ybase where the result needs it (all of it for an add, the
 *               uncovered pixels for a plain write), reads the block stack where a block covers the pixel and
 *               writes y once.  Same y, every byte moved once.  A list that names a block several times gets
 *               the CPU functor's result here as well (the last of the rows wins a plain write, an add sums
 *               all of them in list order).  A planar stack (transpose=1) is staged through LDS by the same
 *               kernel when bsize[1] and bstride[1] are multiples of 4, bstride[1] divides the kernel's strip
 *               width (256 channel vectors, i.e. 32 pixels at 32 channels or more) and boffset[1] is a
 *               multiple of bstride[1]; other planar geometries whose blocks tile the plane (bsize == bstride,
 *               cells of 4 KB or more) are built by one launch over the cells of the block grid (a cell with a
 *               block from the stack, an empty cell from ybase; exact for repeated rows as well); the remaining
 *               planar geometries take two passes once the blocks cover 16 MB (copy of the uncovered pixels,
 *               then the scatter kernel, which reads ybase where it adds), and copy-then-scatter below that:
 *               in these two cases rows that name the same block race as they do in the reference's GPU
 *               kernels.  Overlapping plain writes (add=0, bstride < bsize) from
 *               16 MB of blocks on use the owner map of (0) as their coverage record in the same way.
 *               (2) add=1, atomic=1: with it the overlapping adds need no atomics:
 *               - transpose=0 and at most 2x2 blocks per pixel: each pixel is summed by one owner in ascending
 *                 block-list order, bit-identical to the reference's sequential CPU functor;
 *               - otherwise (transpose=1, or up to 16 blocks per pixel): ceil(R/U)*ceil(S/V) passes of plain
 *                 adds, one class of mutually non-overlapping blocks per pass; reproducible, equal to the
 *                 sequential sums up to fp32 reassociation.
 *               Both run at streaming speed, several times faster than hardware atomics.  Without scratch, or
 *               when the list names a block twice, hardware fp32 atomics are used: same sums up to fp32
 *               reassociation, in no particular order.
 */
int sbnet_sparse_scatter(const float* x, int32_t num_active, const int16_t* active_block_indices,
                         const float* ybase, const int64_t* ybase_dims, int ybase_rank,
                         const int32_t* bsize, int bsize_len,
                         const int32_t* bstride, int bstride_len,
                         const int32_t* boffset, int boffset_len,
                         int add, int atomic, int transpose, float* y,
                         void* workspace, size_t workspace_bytes, void* stream);

/* Op level, in place: replaces SparseScatterOp<GPUDevice,float,true>::Compute ("SparseScatterVar",
   sparse_gather.cc:242-254, 335-337).  ybase is modified and is the result. */
int sbnet_sparse_scatter_var(const float* x, int32_t num_active,
                             const int16_t* active_block_indices,
                             float* ybase, const int64_t* ybase_dims, int ybase_rank,
                             const int32_t* bsize, int bsize_len,
                             const int32_t* bstride, int bstride_len,
                             const int32_t* boffset, int boffset_len,
                             int add, int atomic, int transpose,
                             void* workspace, size_t workspace_bytes, void* stream);

/* Functor level: replaces SparseScatterFunctor<GPUDevice,float>::operator()
   (sparse_gather.h:45-66, sparse_gather.cu:158-266).  Scatters into y in place, no validation
   of the add/atomic/overlap combination. */
int sbnet_sparse_scatter_functor(const float* x, int N, int H, int W, int C, float* y,
                                 int bOffsH0, int bOffsW0, int bSzH, int bSzW, int bStrH,
                                 int bStrW, int numActive, const int16_t* activeBlockIndices,
                                 int add, int transpose, int atomic, void* stream);

/* The same with scratch (sbnet_sparse_scatter_workspace_bytes(), as for the op level): overlapping atomic adds run
   without atomics and overlapping plain writes follow the CPU functor's order.  No counterpart in the reference,
   whose functor has no scratch argument; include/sbnet_reference_functors.hpp calls this one with scratch from
   its scratch provider. */
int sbnet_sparse_scatter_functor_ws(const float* x, int N, int H, int W, int C, float* y,
                                    int bOffsH0, int bOffsW0, int bSzH, int bSzW, int bStrH,
                                    int bStrW, int numActive, const int16_t* activeBlockIndices,
                                    int add, int transpose, int atomic,
                                    void* workspace, size_t workspace_bytes, void* stream);

/* Library-managed device scratch for callers that have no allocator at hand (the functor level of the reference
   passes none down, sparse_gather.h:45-66): returns a buffer of at least `bytes` bytes on the current device.  One
   grow-only buffer is kept per (device, stream); calls on one stream run in order, so consecutive calls of ONE
   host thread on that stream may share it: the pointer is good for the library calls that thread makes next on
   that stream, until its next sbnet_scratch_acquire there.  The bookkeeping is thread-safe and no buffer is
   freed before sbnet_shutdown (a buffer that has been outgrown is kept until then, so a pointer handed out
   earlier never dangles), but two host threads that enqueue on the same stream would interleave their launches
   over the one buffer and corrupt each other's scratch: one enqueuing thread per stream, or scratch of the
   caller's own per call (a TensorFlow binding: allocate_temp).  Growing allocates; a request that would have
   to grow while `stream` is being captured returns NULL, as does a failed allocation. */
void* sbnet_scratch_acquire(size_t bytes, void* stream);

/* Frees what the library keeps between calls: the buffers of sbnet_scratch_acquire and the pinned count words of
   threads that have ended.  Optional; waits for the device.  The library can be used again afterwards. */
int sbnet_shutdown(void);

/* Replaces CopyTensorFunctor<GPUDevice,float>::operator() (sparse_gather.h:69-76,
   sparse_gather.cu:268-276) without its stream synchronisation.  count is in floats. */
int sbnet_copy_tensor(float* dst, const float* src, size_t count, void* stream);

/* ------------------------------------------------------------------------------------------
 * Variants that take the block count from device memory
 * ------------------------------------------------------------------------------------------
 * These have no counterpart in the reference, whose gather and scatter read bin_counts from host memory
 * (sparse_gather.cc:190-192, 315-317) and therefore force a device-to-host copy and a stream
 * synchronisation after every reduce_mask.  They are for callers that must not wait on the host: a pipeline
 * captured into a HIP graph, a serving loop that enqueues reduce_mask -> gather -> ... -> scatter without
 * stalling.  bin_counts_device is the int32 that sbnet_reduce_mask leaves in bin_counts_device; max_active is
 * the capacity of the list and of the block stack (N*bcount[0]*bcount[1] always suffices): the launch is sized
 * for max_active blocks and workgroups of blocks at or beyond *bin_counts_device return at once.  Only the
 * first *bin_counts_device blocks of y (gather) are written / of x (scatter) are read.  All other arguments,
 * checks and results are those of the entry points without the suffix. */
int sbnet_sparse_gather_device_count(const float* x, const int64_t* x_dims, int x_rank,
                                     const int32_t* bin_counts_device, int32_t max_active,
                                     const int16_t* active_block_indices,
                                     const int32_t* bsize, int bsize_len,
                                     const int32_t* bstride, int bstride_len,
                                     const int32_t* boffset, int boffset_len,
                                     int transpose, float* y, void* stream);
int sbnet_sparse_scatter_device_count(const float* x, const int32_t* bin_counts_device, int32_t max_active,
                                      const int16_t* active_block_indices,
                                      const float* ybase, const int64_t* ybase_dims, int ybase_rank,
                                      const int32_t* bsize, int bsize_len,
                                      const int32_t* bstride, int bstride_len,
                                      const int32_t* boffset, int boffset_len,
                                      int add, int atomic, int transpose, float* y,
                                      void* workspace, size_t workspace_bytes, void* stream);
int sbnet_sparse_scatter_var_device_count(const float* x, const int32_t* bin_counts_device, int32_t max_active,
                                          const int16_t* active_block_indices,
                                          float* ybase, const int64_t* ybase_dims, int ybase_rank,
                                          const int32_t* bsize, int bsize_len,
                                          const int32_t* bstride, int bstride_len,
                                          const int32_t* boffset, int boffset_len,
                                          int add, int atomic, int transpose,
                                          void* workspace, size_t workspace_bytes, void* stream);

/* Device timers: replace the CudaTimerStart / CudaTimerEnd ops (sparse_gather.cc:390-469) that the
 * reference's benchmarks bracket their timed regions with.
 *   sbnet_timer_start  creates an event, records it on `stream` and returns it as an opaque 64-bit handle
 *                      (the reference passes the event to the end op the same way, as an int64 tensor).
 *   sbnet_timer_end    records a second event on `stream`, waits for it, writes the elapsed device time in
 *                      milliseconds to *dt_ms and destroys both events; a handle is good for one call.
 * The reference records on the legacy default stream; pass NULL for that. */
int sbnet_timer_start(void* stream, int64_t* start_event);
int sbnet_timer_end(int64_t start_event, void* stream, float* dt_ms);

#ifdef __cplusplus
}
#endif
#endif /* SBNET_AMD_H */
