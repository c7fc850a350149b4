// The reference's GPU functors, specialised by include/sbnet_reference_functors.hpp, run on a real device and
// compared with the CPU oracle: reduce_mask -> sparse_gather -> sparse_scatter exactly as the reference's
// OpKernels call them (reduce_mask.cc:176, sparse_gather.cc:211, 345, 350), both stack layouts.
// Exit status 0 and the line "functor shim gpu ok" mean bit-exact agreement.
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <utility>
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
    const hipStream_t* getStream(const Device& d);
};

struct GpuDevice {
    hipStream_t s;
    const hipStream_t& stream() const { return s; }
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
    if (CopyTensorFunctor<GpuDevice, float>().getStream(d) != &d.s) { std::printf("getStream\n"); return 4; }

    // Overlapping blocks (16x16 at stride 8, every pixel under up to four blocks, as in the atomic scatter-add
    // benchmark configuration) from a shuffled list with different values per block.  The functor header fetches
    // scratch from its provider, so add + atomic runs without atomics in list order and plain writes let the block
    // listed last win: both must equal the sequential CPU functor bit for bit.
    {
        const int oN = 2, oH = 64, oW = 72, oC = 16, oR = 16, oS = 16, oU = 8, oV = 8;
        const int cH = 1 + (oH - 1) / oU, cW = 1 + (oW - 1) / oV;
        std::vector<int16_t> oIdx;
        for (int n = 0; n < oN; ++n)
            for (int bh = 0; bh < cH; ++bh)
                for (int bw = 0; bw < cW; ++bw)
                    if (rnd() > 0.2f) { oIdx.push_back((int16_t)n); oIdx.push_back((int16_t)bh); oIdx.push_back((int16_t)bw); }
        const int oM = (int)oIdx.size() / 3;
        for (int i = oM - 1; i > 0; --i) {  // shuffle rows
            st = st * 1664525u + 1013904223u;
            const int j = (int)((st >> 8) % (unsigned)(i + 1));
            for (int k = 0; k < 3; ++k) std::swap(oIdx[(size_t)i * 3 + k], oIdx[(size_t)j * 3 + k]);
        }
        const size_t sFloats = (size_t)oM * oR * oS * oC, bFloats = (size_t)oN * oH * oW * oC;
        std::vector<float> oStack(sFloats), oBase(bFloats), got(bFloats), ref(bFloats);
        for (auto& v : oStack) v = rnd();
        for (auto& v : oBase) v = rnd();
        float *dS2, *dB2;
        int16_t* dI2;
        CK(hipMalloc((void**)&dS2, sFloats * 4));
        CK(hipMalloc((void**)&dB2, bFloats * 4));
        CK(hipMalloc((void**)&dI2, oIdx.size() * 2));
        CK(hipMemcpy(dS2, oStack.data(), sFloats * 4, hipMemcpyHostToDevice));
        CK(hipMemcpy(dI2, oIdx.data(), oIdx.size() * 2, hipMemcpyHostToDevice));
        for (int mode = 0; mode < 2; ++mode) {  // 0: add + atomic, 1: plain writes
            for (int transpose = 0; transpose < 2; ++transpose) {
                if (mode == 0 && transpose) continue;  // the planar stack adds in passes: equal only up to rounding
                CK(hipMemcpy(dB2, oBase.data(), bFloats * 4, hipMemcpyHostToDevice));
                SparseScatterFunctor<GpuDevice, float>()(d, dS2, oN, oH, oW, oC, dB2, 0, 0, oR, oS, oU, oV, oM, dI2,
                                                         mode == 0, transpose != 0, mode == 0);
                CK(hipStreamSynchronize(d.s));
                CK(hipMemcpy(got.data(), dB2, bFloats * 4, hipMemcpyDeviceToHost));
                ref = oBase;
                oracle_sparse_scatter(oStack.data(), oN, oH, oW, oC, ref.data(), 0, 0, oR, oS, oU, oV, oM, oIdx.data(),
                                      mode == 0, transpose, mode == 0);
                if (std::memcmp(got.data(), ref.data(), bFloats * 4) != 0) {
                    std::printf("overlapping scatter differs (mode=%d transpose=%d)\n", mode, transpose);
                    return 5;
                }
            }
        }
    }
    if (sbnet_shutdown() != SBNET_OK) { std::printf("sbnet_shutdown\n"); return 6; }
    std::printf("functor shim gpu ok: %d of %d blocks active\n", M, T);
    return 0;
}
