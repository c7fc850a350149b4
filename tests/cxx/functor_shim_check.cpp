// Compiles include/sbnet_reference_functors.hpp the way a build of the reference would: the four functor
// templates are declared first (here with the operator() signatures of reduce_mask.h:23-44 and
// sparse_gather.h:23-76, nothing else), a device type with stream() stands in for Eigen::GpuDevice, and the
// macro supplies the GPU specialisations.  Every call below fails the library's argument validation before
// any device work, so the program runs without a GPU; it checks that each functor reaches the library and
// that a failure reaches the error handler.
#include <cstring>
#include <cstdio>

template <typename Device, typename T> struct ReduceMaskFunctor {
    void operator()(const Device& d, const T* mask, int N, int H, int W, float threshold, int bOffsH0, int bOffsW0,
                    int bSzH, int bSzW, int bStrH, int bStrW, int bCntH, int bCntW, unsigned int numBins,
                    unsigned int binSize, short* activeBlockIndices, int* binCounts, bool avgPool);
};
template <typename Device, typename T> struct SparseGatherFunctor {
    void operator()(const Device& d, const T* x, int N, int H, int W, int C, T* y, int bOffsH0, int bOffsW0, int bSzH,
                    int bSzW, int bStrH, int bStrW, int numActive, const short* activeBlockIndices, bool transpose);
};
template <typename Device, typename T> struct SparseScatterFunctor {
    void operator()(const Device& d, const T* x, int N, int H, int W, int C, T* y, int bOffsH0, int bOffsW0, int bSzH,
                    int bSzW, int bStrH, int bStrW, int numActive, const short* activeBlockIndices, bool add,
                    bool transpose, bool atomic);
};
template <typename Device, typename T> struct CopyTensorFunctor {
    void operator()(const Device& d, T* dst, const T* src, int count);
    void** getStream(const Device& d);
};

struct FakeGpuDevice {
    void* s;
    void* const& stream() const { return s; }  // a reference, as Eigen::GpuDevice::stream() returns
};

#include "sbnet_reference_functors.hpp"

SBNET_AMD_GPU_FUNCTORS(FakeGpuDevice)

static int g_calls = 0, g_last = 0;
static char g_what[64];
static void record(int status, const char* what)
{
    ++g_calls;
    g_last = status;
    std::strncpy(g_what, what, sizeof(g_what) - 1);
}

int main()
{
    sbnet_amd::error_handler() = record;
    FakeGpuDevice d = {nullptr};
    const float* nof = nullptr;
    ReduceMaskFunctor<FakeGpuDevice, float>()(d, nof, 1, 8, 8, 0.5f, 0, 0, 2, 2, 2, 2, 4, 4, 1, 1, nullptr, nullptr, false);
    if (g_calls != 1 || g_last != SBNET_EINVAL_ARG || std::strcmp(g_what, "ReduceMaskFunctor")) return 1;
    SparseGatherFunctor<FakeGpuDevice, float>()(d, nof, 1, 8, 8, 4, nullptr, 0, 0, 2, 2, 2, 2, 3, nullptr, true);
    if (g_calls != 2 || g_last != SBNET_EINVAL_ARG || std::strcmp(g_what, "SparseGatherFunctor")) return 2;
    SparseScatterFunctor<FakeGpuDevice, float>()(d, nof, 1, 8, 8, 4, nullptr, 0, 0, 2, 2, 2, 2, 3, nullptr, true, false,
                                                 false);
    if (g_calls != 3 || g_last != SBNET_EINVAL_ARG || std::strcmp(g_what, "SparseScatterFunctor")) return 3;
    CopyTensorFunctor<FakeGpuDevice, float>()(d, nullptr, nof, 16);
    if (g_calls != 4 || g_last != SBNET_EINVAL_ARG || std::strcmp(g_what, "CopyTensorFunctor")) return 4;
    // nothing to do is not an error
    SparseGatherFunctor<FakeGpuDevice, float>()(d, nof, 1, 8, 8, 4, nullptr, 0, 0, 2, 2, 2, 2, 0, nullptr, false);
    CopyTensorFunctor<FakeGpuDevice, float>()(d, nullptr, nof, 0);
    if (g_calls != 4) return 5;
    // getStream hands out the address of the device's stream handle (sparse_gather.cu:275)
    if (CopyTensorFunctor<FakeGpuDevice, float>().getStream(d) != &d.s) return 6;
    // a scratch provider of the caller's replaces the library's
    sbnet_amd::scratch_provider() = [](size_t, void*) -> void* { ++g_calls; return nullptr; };
    SparseScatterFunctor<FakeGpuDevice, float>()(d, nof, 1, 8, 8, 4, nullptr, 0, 0, 2, 2, 2, 2, 3, nullptr, true, false,
                                                 true);
    if (g_calls != 6 || g_last != SBNET_EINVAL_ARG) return 7;  // one call of the provider, one of the handler
    std::printf("functor shim ok\n");
    return 0;
}
