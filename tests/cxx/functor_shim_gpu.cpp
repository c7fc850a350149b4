// The reference's GPU functors, specialised by include/sbnet_reference_functors.hpp, run on a real device and
// compared with the CPU oracle: reduce_mask -> sparse_gather -> sparse_scatter exactly as the reference's
// OpKernels call them (reduce_mask.cc:176, sparse_gather.cc:211, 345, 350), both stack layouts.
// Exit status 0 and the line "functor shim gpu ok" mean bit-exact agreement.
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

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
};

struct GpuDevice {
    hipStream_t s;
    hipStream_t stream() const { return s; }
};

#include "sbnet_reference_functors.hpp"

SBNET_AMD_GPU_FUNCTORS(GpuDevice)

// the CPU oracle (oracle/sbnet_oracle.c)
extern "C" {
int oracle_reduce_mask_functor(const float* mask, int N, int H, int W, float threshold, int bOffsH0, int bOffsW0,
                               int bSzH, int bSzW, int bStrH, int bStrW, int bCntH, int bCntW,
                               int16_t* activeBlockIndices, int avgPool);
void oracle_sparse_gather(const float* x, int N, int H, int W, int C, float* y, int bOffsH0, int bOffsW0, int bSzH,
                          int bSzW, int bStrH, int bStrW, int numActive, const int16_t* activeBlockIndices,
                          int transpose);
void oracle_sparse_scatter(const float* x, int N, int H, int W, int C, float* y, int bOffsH0, int bOffsW0, int bSzH,
                           int bSzW, int bStrH, int bStrW, int numActive, const int16_t* activeBlockIndices, int add,
                           int transpose, int atomic);
}

#define CK(call)                                                                             \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess) {                                                              \
            std::printf("%s: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__);       \
            return 10;                                                                       \
        }                                                                                    \
    } while (0)

int main()
{
    const int N = 2, H = 45, W = 52, C = 24;
    const int R = 9, S = 7, U = 8, V = 6, oh = -1, ow = -2;
    const int bCntH = 1 + (H - oh - 1) / U, bCntW = 1 + (W - ow - 1) / V;
    const int T = N * bCntH * bCntW;
    std::vector<float> mask((size_t)N * H * W), x((size_t)N * H * W * C), base(x.size());
    unsigned st = 2024u;
    auto rnd = [&]() { st = st * 1664525u + 1013904223u; return (float)((int)(st >> 9) % 2001 - 1000) * 1e-3f; };
    for (auto& v : mask) v = rnd();
    for (auto& v : x) v = rnd();
    for (auto& v : base) v = rnd();
    const float tol = 0.97f;  // max pooling over 63 pixels: about 60 % of the blocks are active

    std::vector<int16_t> idxRef((size_t)T * 3);
    const int M = oracle_reduce_mask_functor(mask.data(), N, H, W, tol, oh, ow, R, S, U, V, bCntH, bCntW, idxRef.data(), 0);
    if (M <= 0 || M >= T) { std::printf("degenerate mask: %d of %d\n", M, T); return 11; }

    GpuDevice d;
    CK(hipStreamCreate(&d.s));
    float *dMask, *dX, *dBase, *dY, *dStack;
    int16_t* dIdx;
    int* dCount;
    const size_t stackFloats = (size_t)M * R * S * C;
    CK(hipMalloc((void**)&dMask, mask.size() * 4));
    CK(hipMalloc((void**)&dX, x.size() * 4));
    CK(hipMalloc((void**)&dBase, x.size() * 4));
    CK(hipMalloc((void**)&dY, x.size() * 4));
    CK(hipMalloc((void**)&dStack, stackFloats * 4));
    CK(hipMalloc((void**)&dIdx, (size_t)T * 6));
    CK(hipMalloc((void**)&dCount, 4));
    CK(hipMemcpy(dMask, mask.data(), mask.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(dX, x.data(), x.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(dBase, base.data(), base.size() * 4, hipMemcpyHostToDevice));

    ReduceMaskFunctor<GpuDevice, float>()(d, dMask, N, H, W, tol, oh, ow, R, S, U, V, bCntH, bCntW, 1, 1, dIdx, dCount, false);
    int count = -1;
    std::vector<int16_t> idx((size_t)T * 3);
    CK(hipStreamSynchronize(d.s));
    CK(hipMemcpy(&count, dCount, 4, hipMemcpyDeviceToHost));
    CK(hipMemcpy(idx.data(), dIdx, (size_t)T * 6, hipMemcpyDeviceToHost));
    if (count != M || std::memcmp(idx.data(), idxRef.data(), (size_t)M * 6) != 0) {
        std::printf("reduce_mask differs: count %d, oracle %d\n", count, M);
        return 1;
    }

    std::vector<float> stack(stackFloats), stackRef(stackFloats), y(x.size()), yRef(x.size());
    for (int transpose = 0; transpose < 2; ++transpose) {
        SparseGatherFunctor<GpuDevice, float>()(d, dX, N, H, W, C, dStack, oh, ow, R, S, U, V, M, dIdx, transpose != 0);
        CK(hipStreamSynchronize(d.s));
        CK(hipMemcpy(stack.data(), dStack, stackFloats * 4, hipMemcpyDeviceToHost));
        oracle_sparse_gather(x.data(), N, H, W, C, stackRef.data(), oh, ow, R, S, U, V, M, idxRef.data(), transpose);
        if (std::memcmp(stack.data(), stackRef.data(), stackFloats * 4) != 0) {
            std::printf("gather differs (transpose=%d)\n", transpose);
            return 2;
        }
        // copy of the base, then the blocks written on top (overlapping blocks carry equal values)
        CopyTensorFunctor<GpuDevice, float>()(d, dY, dBase, (int)x.size());
        SparseScatterFunctor<GpuDevice, float>()(d, dStack, N, H, W, C, dY, oh, ow, R, S, U, V, M, dIdx, false,
                                                 transpose != 0, false);
        CK(hipStreamSynchronize(d.s));
        CK(hipMemcpy(y.data(), dY, x.size() * 4, hipMemcpyDeviceToHost));
        yRef = base;
        oracle_sparse_scatter(stackRef.data(), N, H, W, C, yRef.data(), oh, ow, R, S, U, V, M, idxRef.data(), 0, transpose, 0);
        if (std::memcmp(y.data(), yRef.data(), x.size() * 4) != 0) {
            std::printf("scatter differs (transpose=%d)\n", transpose);
            return 3;
        }
    }
    std::printf("functor shim gpu ok: %d of %d blocks active\n", M, T);
    return 0;
}
