/*
 * sbnet_reference_functors.hpp -- the reference's GPU functors on top of libsbnet_amd.so.
 *
 * The reference splits each op into an OpKernel (reduce_mask.cc, sparse_gather.cc) and a functor template
 * declared in reduce_mask.h:23-44 and sparse_gather.h:23-76.  The OpKernels call
 *     ReduceMaskFunctor<Device, T>()(d, mask, N, H, W, ...)            reduce_mask.cc:176
 *     SparseGatherFunctor<Device, T>()(d, x, N, H, W, C, y, ...)       sparse_gather.cc:211
 *     CopyTensorFunctor<Device, T>()(d, dst, src, count)               sparse_gather.cc:345
 *     SparseScatterFunctor<Device, T>()(d, x, N, H, W, C, y, ...)      sparse_gather.cc:350
 * and the GPUDevice specialisations live in reduce_mask.cu:39-93 and sparse_gather.cu:62-280, each closed by
 * an explicit instantiation for float.  This header provides those specialisations, so that one source file
 *
 *     #include "reduce_mask.h"
 *     #include "sparse_gather.h"
 *     #include "sbnet_reference_functors.hpp"
 *     typedef Eigen::GpuDevice GPUDevice;
 *     SBNET_AMD_GPU_FUNCTORS(GPUDevice)
 *
 * replaces both .cu files and the OpKernels compile unchanged.  `Device` only has to offer stream(), returning
 * a reference to the HIP stream the op must run on (Eigen::GpuDevice does; getStream hands out its address).  The primary templates must be declared before
 * the macro is used; this header does not declare them.
 *
 * Differences from the .cu files it replaces, all inherited from the library: block indices come out in
 * (n, bh, bw) order, avg pooling decides as the CPU functor does, CopyTensorFunctor does not synchronise the
 * stream.  The functors return void, as in the reference; a failing call goes to the error handler, which by
 * default prints the library's message and aborts (the reference prints and exits, op_utils.h:27-35).
 */
#ifndef SBNET_REFERENCE_FUNCTORS_HPP
#define SBNET_REFERENCE_FUNCTORS_HPP

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "sbnet_amd.h"

namespace sbnet_amd {

typedef void (*ErrorHandler)(int status, const char* what);

inline void default_error_handler(int status, const char* what)
{
    std::fprintf(stderr, "sbnet_amd: %s failed: %s (status %d, hipError_t %d)\n", what, sbnet_status_string(status),
                 status, sbnet_last_hip_error());
    std::abort();
}

inline ErrorHandler& error_handler()
{
    static ErrorHandler h = default_error_handler;
    return h;
}

inline void check(int status, const char* what)
{
    if (status != SBNET_OK) error_handler()(status, what);
}

template <typename Device> inline void* stream_of(const Device& d) { return (void*)d.stream(); }

// Device scratch for the functors.  The reference's functor signatures carry no scratch, but the fast paths of
// the library need some (reduce_mask's flags; the atomic-free overlapping scatter-add; ordered overlapping
// writes).  A provider returns at least `bytes` bytes valid until its next call on the same stream, or NULL
// (the functors then take the paths that need none).  The default is the library's own per-stream buffer; a
// framework with a stream-ordered allocator can install its own.
typedef void* (*ScratchProvider)(size_t bytes, void* stream);

inline ScratchProvider& scratch_provider()
{
    static ScratchProvider p = sbnet_scratch_acquire;
    return p;
}

inline void* scratch(size_t bytes, void* stream)
{
    return (bytes && scratch_provider()) ? scratch_provider()(bytes, stream) : NULL;
}

}  // namespace sbnet_amd

#define SBNET_AMD_GPU_FUNCTORS(DEVICE)                                                                              \
    template <typename T> struct ReduceMaskFunctor<DEVICE, T> {                                                     \
        void operator()(const DEVICE& d, const T* mask, int N, int H, int W, float threshold, int bOffsH0,          \
                        int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int bCntH, int bCntW,                \
                        unsigned int numBins, unsigned int binSize, short* activeBlockIndices, int* binCounts,      \
                        bool avgPool)                                                                               \
        {                                                                                                           \
            const int32_t bcount_[2] = {bCntH, bCntW};                                                              \
            const size_t need_ = sbnet_reduce_mask_workspace_bytes(N, bcount_, 2);                                  \
            void* ws_ = sbnet_amd::scratch(need_, sbnet_amd::stream_of(d));                                         \
            /* without scratch the library allocates and frees its own for the call */                              \
            sbnet_amd::check(sbnet_reduce_mask_functor(mask, N, H, W, threshold, bOffsH0, bOffsW0, bSzH, bSzW,      \
                                                       bStrH, bStrW, bCntH, bCntW, numBins, binSize,                \
                                                       activeBlockIndices, binCounts, avgPool ? 1 : 0, ws_,         \
                                                       ws_ ? need_ : 0, sbnet_amd::stream_of(d)),                   \
                             "ReduceMaskFunctor");                                                                  \
        }                                                                                                           \
    };                                                                                                              \
    template <typename T> struct SparseGatherFunctor<DEVICE, T> {                                                   \
        void operator()(const DEVICE& d, const T* x, int N, int H, int W, int C, T* y, int bOffsH0, int bOffsW0,    \
                        int bSzH, int bSzW, int bStrH, int bStrW, int numActive, const short* activeBlockIndices,   \
                        bool transpose)                                                                             \
        {                                                                                                           \
            sbnet_amd::check(sbnet_sparse_gather_functor(x, N, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH,     \
                                                         bStrW, numActive, activeBlockIndices, transpose ? 1 : 0,   \
                                                         sbnet_amd::stream_of(d)),                                  \
                             "SparseGatherFunctor");                                                                \
        }                                                                                                           \
    };                                                                                                              \
    template <typename T> struct SparseScatterFunctor<DEVICE, T> {                                                  \
        void operator()(const DEVICE& d, const T* x, int N, int H, int W, int C, T* y, int bOffsH0, int bOffsW0,    \
                        int bSzH, int bSzW, int bStrH, int bStrW, int numActive, const short* activeBlockIndices,   \
                        bool add, bool transpose, bool atomic)                                                      \
        {                                                                                                           \
            size_t need_ = 0;                                                                                       \
            if ((add && atomic) || (!add && (bStrH < bSzH || bStrW < bSzW))) {                                      \
                const int64_t dims_[4] = {N, H, W, C};                                                              \
                const int32_t bsize_[2] = {bSzH, bSzW}, bstride_[2] = {bStrH, bStrW},                               \
                              boffset_[2] = {bOffsH0, bOffsW0};                                                     \
                need_ = sbnet_sparse_scatter_workspace_bytes(numActive, dims_, 4, bsize_, 2, bstride_, 2,           \
                                                             boffset_, 2);                                          \
            }                                                                                                       \
            void* ws_ = sbnet_amd::scratch(need_, sbnet_amd::stream_of(d));                                         \
            sbnet_amd::check(sbnet_sparse_scatter_functor_ws(x, N, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW,        \
                                                             bStrH, bStrW, numActive, activeBlockIndices,           \
                                                             add ? 1 : 0, transpose ? 1 : 0, atomic ? 1 : 0, ws_,   \
                                                             ws_ ? need_ : 0, sbnet_amd::stream_of(d)),             \
                             "SparseScatterFunctor");                                                               \
        }                                                                                                           \
    };                                                                                                              \
    template <typename T> struct CopyTensorFunctor<DEVICE, T> {                                                     \
        void operator()(const DEVICE& d, T* dst, const T* src, int count)                                           \
        {                                                                                                           \
            sbnet_amd::check(sbnet_copy_tensor(dst, src, (size_t)count, sbnet_amd::stream_of(d)),                   \
                             "CopyTensorFunctor");                                                                  \
        }                                                                                                           \
        /* sparse_gather.h:75, sparse_gather.cu:275: the address of the device's stream handle */                   \
        auto getStream(const DEVICE& d) -> decltype(&d.stream()) { return &d.stream(); }                            \
    };                                                                                                              \
    template struct ReduceMaskFunctor<DEVICE, float>;                                                               \
    template struct SparseGatherFunctor<DEVICE, float>;                                                             \
    template struct SparseScatterFunctor<DEVICE, float>;                                                            \
    template struct CopyTensorFunctor<DEVICE, float>;

#endif /* SBNET_REFERENCE_FUNCTORS_HPP */
