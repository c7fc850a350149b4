// reduce_mask on gfx950: pooling, ordered stream compaction, the count handed to the host, and the library's own
// static scratch.  Reference semantics: sbnet_tensorflow/sbnet_ops/reduce_mask.cc:68-96, 206-218.
#include "sbnet_device.h"

namespace sbnet {

// ---------------------------------------------------------------------------------------------
// reduce_mask: pooling + ordered stream compaction
// ---------------------------------------------------------------------------------------------
//
// Kernel 1 (k_reduce_pool): G = 2^logG lanes cooperate on one sparsity block (G grows with the
// window, from 1 lane for tiny windows to a full wave), decide "active" and store one flag byte
// per block plus one count per workgroup.  Blocks are numbered b = (n*bCntH + bh)*bCntW + bw,
// the order in which the CPU functor visits them (reduce_mask.cc:71-73).
//
// Kernel 2 (k_reduce_compact): one thread per block; wave64 ballot + popcount gives the rank of
// each active block inside its wave, LDS the wave offsets, the per-workgroup counts of kernel 1
// the offset of the workgroup (summed by each workgroup while there are few; beyond
// SCAN_MIN_COUNTS counts k_reduce_scan, one workgroup, turns them into exclusive prefix sums
// first).  Triples therefore land in the CPU functor's order, and the last workgroup knows the
// total: it stores the count and applies the "no active block" fix-up (reduce_mask.cc:206-218)
// on the device.  Nothing in the scratch has to be cleared before a call: every byte that is
// read has been written by the same call.
//
// (A single launch, in which every workgroup publishes its bits in tagged words and the last one
// to publish compacts, was measured and dropped: workgroups of one launch can only meet through
// device-scope memory operations, and on this chip one such load takes about 2 us: 7.9 us per
// launch against 6.7 us for the two launches; device-scope fences instead of atomic accesses
// cost 30 us.)
//
// avg mode: the CPU functor adds the in-range pixels in row-major order (reduce_mask.cc:78-88)
// and fp32 addition is not associative.  A cooperative sum is used only where it provably yields
// the same decision: (a) all values are integers and sum|v| < 2^24, so every order is exact;
// (b) the interval [sum-E, sum+E], E bounding the difference between any two summation orders,
// lies on one side of the threshold after the (monotonic, correctly rounded) division.  Otherwise
// one lane redoes the sum in the reference order.

struct PoolArgs {
    int N, H, W;
    int R, S, U, V, oh, ow;
    int bCntH, bCntW;
    uint32_t T;       // N * bCntH * bCntW
    float tol;
    int avg;
    int logG;         // log2 of the lanes that share one block
    int passes;       // blocks per group
    FastDiv dBw, dBhw;
};

constexpr uint32_t SCAN_MIN_COUNTS = 1024;

// Stores the count (and, for an empty list, the (0,0,0) triple of reduce_mask.cc:206-218) and hands it to a
// polling host: one 8-byte store (sequence number, count) into pinned host memory; system scope, so it leaves
// the device at once.
__device__ __forceinline__ void publish_count(int total, int fixupZero, int16_t* __restrict__ idx,
                                              int32_t* __restrict__ binCount, unsigned long long* hostSignal,
                                              uint32_t hostSeq)
{
    if (total == 0 && fixupZero) {
        idx[0] = 0; idx[1] = 0; idx[2] = 0;
        total = 1;
    }
    *binCount = total;
    // (relaxed: the host takes nothing but this word from the device; a release here would first write back the L2)
    if (hostSignal)
        __hip_atomic_store(hostSignal, ((unsigned long long)hostSeq << 32) | (uint32_t)total, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ float next_down(float f)
{
    if (!(f == f) || f == -INFINITY) return f;
    if (f == 0.f) return -1.401298464e-45f;
    int i = __float_as_int(f);
    i += (f > 0.f) ? -1 : 1;
    return __int_as_float(i);
}

__device__ __forceinline__ float next_up(float f) { return -next_down(-f); }

constexpr int POOL_LD = 12;  // loads in flight per lane (a 6x6 window over 4 lanes is 9 loads each: one round, not 8 + 1)

__global__ __launch_bounds__(256) void k_reduce_pool(const float* __restrict__ mask, PoolArgs a,
                                                     uint8_t* __restrict__ flags, int32_t* __restrict__ counts)
{
    __shared__ int wgCount;
    const uint32_t tid = threadIdx.x;
    if (tid == 0) wgCount = 0;
    __syncthreads();

    const int G = 1 << a.logG;
    const uint32_t groups = 256u >> a.logG;
    const uint32_t grp = tid >> a.logG;
    const int l = (int)(tid & (uint32_t)(G - 1));
    const uint32_t CH = groups * (uint32_t)a.passes;
    const float denom = (float)(a.R * a.S);

    for (int pass = 0; pass < a.passes; ++pass) {
        const uint32_t b = blockIdx.x * CH + (uint32_t)pass * groups + grp;
        const bool live = b < a.T;
        int n = 0, hlo = 0, hhi = 0, wlo = 0, whi = 0;
        if (live) {
            n = (int)fdiv(b, a.dBhw);
            const uint32_t rem = b - (uint32_t)n * (uint32_t)(a.bCntH * a.bCntW);
            const int bh = (int)fdiv(rem, a.dBw);
            const int bw = (int)(rem - (uint32_t)bh * (uint32_t)a.bCntW);
            const int h0 = a.oh + bh * a.U, w0 = a.ow + bw * a.V;
            hlo = max(0, h0); hhi = min(a.H, h0 + a.R);
            wlo = max(0, w0); whi = min(a.W, w0 + a.S);
        }
        const float* __restrict__ img = mask + (int64_t)n * a.H * a.W;
        float sum = 0.f, sabs = 0.f;
        int allint = 1, any = 0;
        // The clipped window, flattened row-major, is dealt to the G lanes in turn; POOL_LD loads per lane go
        // out back to back before the first one is used (the window is a handful of cache lines per lane, so
        // the kernel is a chain of load latencies and nothing else).  Lanes past the end read element 0 of
        // the window's first row, which exists whenever the window is not empty.
        const uint32_t cw = (uint32_t)max(0, whi - wlo), chh = (uint32_t)max(0, hhi - hlo);
        const uint32_t npxc = cw * chh;  // below 2^31: the host checks R*S
        const float* __restrict__ win = img + (int64_t)hlo * a.W + wlo;
        const uint32_t stepR = (uint32_t)G / max(cw, 1u), stepS = (uint32_t)G - stepR * cw;
        uint32_t r = (uint32_t)l / max(cw, 1u), sc = (uint32_t)l - r * cw;
        for (uint32_t e0 = (uint32_t)l; e0 < npxc; e0 += POOL_LD * (uint32_t)G) {
            float v[POOL_LD];
            bool ok[POOL_LD];
#pragma unroll
            for (int k = 0; k < POOL_LD; ++k) {
                ok[k] = e0 + (uint32_t)k * (uint32_t)G < npxc;
                v[k] = win[ok[k] ? (int64_t)r * a.W + sc : 0];
                sc += stepS;
                r += stepR;
                if (sc >= cw) {
                    sc -= cw;
                    ++r;
                }
            }
#pragma unroll
            for (int k = 0; k < POOL_LD; ++k) {
                if (a.avg) {
                    const float t = ok[k] ? v[k] : 0.f;
                    sum += t;
                    sabs += fabsf(t);
                    allint &= (t == truncf(t));
                } else {
                    any |= (ok[k] && v[k] > a.tol);
                }
            }
        }
        // butterfly over the G lanes of the group: every lane ends with the same values
        for (int off = 1; off < G; off <<= 1) {
            sum += __shfl_xor(sum, off);
            sabs += __shfl_xor(sabs, off);
            allint &= __shfl_xor(allint, off);
            any |= __shfl_xor(any, off);
        }
        if (live && l == 0) {
            bool act;
            if (!a.avg) {
                act = any != 0;
            } else {
                bool decided = false;
                act = false;
                if (G == 1 || (allint && sabs < 16777216.f)) {
                    act = (sum / denom) > a.tol;
                    decided = true;
                } else {
                    const int npx = max(0, hhi - hlo) * max(0, whi - wlo);
                    if (npx <= (1 << 20)) {
                        // |sum_a - sum_b| <= 2*gamma(n-1)*sum|v| for any two orders a, b
                        const float E = sabs * ((float)npx * 1.4901161e-7f);  // 2.5 * n * 2^-24
                        const float lo = next_down(sum - E), hi = next_up(sum + E);
                        const bool alo = (lo / denom) > a.tol, ahi = (hi / denom) > a.tol;
                        if (alo == ahi && lo == lo && hi == hi) { act = alo; decided = true; }
                    }
                }
                if (!decided) {
                    float s = 0.f;
                    for (int hh = hlo; hh < hhi; ++hh) {
                        const float* __restrict__ row = img + (int64_t)hh * a.W;
                        for (int ww = wlo; ww < whi; ++ww) s += row[ww];
                    }
                    act = (s / denom) > a.tol;
                }
            }
            flags[b] = act ? 1 : 0;
            if (act) atomicAdd(&wgCount, 1);
        }
    }
    __syncthreads();
    if (tid == 0) counts[blockIdx.x] = wgCount;
}

// Exclusive prefix sums of the pooling workgroups' counts, in place, by one workgroup of 1024 threads: each
// thread sums a contiguous piece, the pieces are scanned through LDS, and each thread rewrites its piece.
__global__ __launch_bounds__(1024) void k_reduce_scan(int32_t* __restrict__ counts, uint32_t n)
{
    __shared__ int part[1024];
    const uint32_t tid = threadIdx.x;
    const uint32_t per = (n + 1023u) / 1024u;
    const uint32_t lo = min(tid * per, n), hi = min(lo + per, n);
    int sum = 0;
    for (uint32_t i = lo; i < hi; ++i) sum += counts[i];
    part[tid] = sum;
    __syncthreads();
    for (uint32_t off = 1; off < 1024u; off <<= 1) {
        const int add = tid >= off ? part[tid - off] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int run = part[tid] - sum;
    for (uint32_t i = lo; i < hi; ++i) {
        const int c = counts[i];
        counts[i] = run;
        run += c;
    }
}

struct CompactArgs {
    uint32_t T;
    uint32_t nCounts;   // pooling workgroups
    uint32_t ratio;     // pooling workgroups per 256 blocks
    int scanned;        // counts already hold exclusive prefix sums (k_reduce_scan has run)
    int bCntH, bCntW;
    int fixupZero;
    FastDiv dBw, dBhw;
};

__global__ __launch_bounds__(256) void k_reduce_compact(const uint8_t* __restrict__ flags,
                                                        const int32_t* __restrict__ counts, CompactArgs a,
                                                        int16_t* __restrict__ idx, int32_t* __restrict__ binCount,
                                                        unsigned long long* hostSignal, uint32_t hostSeq)
{
    __shared__ int waveSum[4];
    __shared__ int waveCnt[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // active blocks before this workgroup's 256 blocks: read from the scanned counts, or (few counts) summed here
    uint32_t nPrev = blockIdx.x * a.ratio;
    if (nPrev > a.nCounts) nPrev = a.nCounts;
    int part = 0;
    if (a.scanned) {
        // (256*blockIdx.x < T, hence nPrev < nCounts: the prefix is there)
        if (tid == 0) part = counts[nPrev];
    } else {
        for (uint32_t i = tid; i < nPrev; i += 256) part += counts[i];
    }
    for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
    if (lane == 0) waveSum[wave] = part;

    const uint32_t b = blockIdx.x * 256u + tid;
    const bool f = (b < a.T) && flags[b] != 0;
    const unsigned long long bal = __ballot(f);
    const int rank = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) waveCnt[wave] = __popcll(bal);
    __syncthreads();

    const int base = waveSum[0] + waveSum[1] + waveSum[2] + waveSum[3];
    int woff = 0;
    for (uint32_t w = 0; w < wave; ++w) woff += waveCnt[w];
    if (f) {
        const uint32_t n = fdiv(b, a.dBhw);
        const uint32_t rem = b - n * (uint32_t)(a.bCntH * a.bCntW);
        const uint32_t bh = fdiv(rem, a.dBw);
        const uint32_t bw = rem - bh * (uint32_t)a.bCntW;
        int16_t* t = idx + (size_t)(base + woff + rank) * 3;
        t[0] = (int16_t)n;
        t[1] = (int16_t)bh;
        t[2] = (int16_t)bw;
    }
    if (blockIdx.x == gridDim.x - 1 && tid == 0)
        publish_count(base + waveCnt[0] + waveCnt[1] + waveCnt[2] + waveCnt[3], a.fixupZero, idx, binCount, hostSignal,
                      hostSeq);
}

// Scratch layout: one flag byte per block (padded to 16), one int32 count per pooling workgroup (one per block
// at worst), and the total for callers that give no device count.
size_t reduce_mask_workspace_bytes(int64_t totalBlocks)
{
    const size_t flags = ((size_t)totalBlocks + 15) & ~(size_t)15;
    return flags + (size_t)totalBlocks * sizeof(int32_t) + 16;
}

int32_t* reduce_mask_count_slot(void* workspace, int64_t totalBlocks)
{
    const size_t flags = ((size_t)totalBlocks + 15) & ~(size_t)15;
    return reinterpret_cast<int32_t*>(static_cast<uint8_t*>(workspace) + flags) + totalBlocks;
}

// Scratch for callers that can neither allocate nor bring a workspace (sbnet_reduce_mask_static): one array per
// GPU, part of the loaded code object, held until the process ends.  Host code never passes the array's name to a
// kernel: the name is a host-side stand-in, the device address comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[STATIC_SCRATCH_BYTES];

hipError_t static_scratch(void** ptr)
{
    constexpr int MAX_DEVICES = 64;
    static std::mutex mutex;
    static void* ptrs[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!ptrs[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // of the current device's copy of the array
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        ptrs[dev] = p;
    }
    *ptr = ptrs[dev];
    return hipSuccess;
}

hipError_t launch_reduce_mask(const float* mask, const Geom& g, int bCntH, int bCntW, float tol,
                              bool avgPool, bool fixupZero, int16_t* activeBlockIndices,
                              int32_t* binCountDevice, void* workspace, hipStream_t stream,
                              unsigned long long* hostSignal, uint32_t hostSeq)
{
    const uint32_t T = (uint32_t)((int64_t)g.N * bCntH * bCntW);
    uint8_t* flags = static_cast<uint8_t*>(workspace);
    const size_t flagBytes = ((size_t)T + 15) & ~(size_t)15;
    int32_t* counts = reinterpret_cast<int32_t*>(flags + flagBytes);
    if (!binCountDevice) binCountDevice = reduce_mask_count_slot(workspace, T);

    PoolArgs p;
    p.N = g.N; p.H = g.H; p.W = g.W;
    p.R = g.R; p.S = g.S; p.U = g.U; p.V = g.V; p.oh = g.oh; p.ow = g.ow;
    p.bCntH = bCntH; p.bCntW = bCntW;
    p.T = T;
    p.tol = tol;
    p.avg = avgPool ? 1 : 0;
    const uint64_t npx = (uint64_t)g.R * (uint64_t)g.S;
    // the kernel counts the pixels of a block's in-image window in 32 bits
    if ((uint64_t)(g.R < g.H ? g.R : g.H) * (uint64_t)(g.S < g.W ? g.S : g.W) >= (1ull << 31)) return hipErrorInvalidValue;
    int logG = npx >= 16 ? ilog2_floor((uint32_t)(npx / 8 > 64 ? 64 : npx / 8)) : 0;
    if (logG > 6) logG = 6;
    p.logG = logG;
    const uint32_t groups = 256u >> logG;
    int passes = 1;
    while (passes < (1 << logG) && passes < 8 && T / (groups * passes) > 2048) passes *= 2;
    p.passes = passes;
    p.dBw = make_fastdiv((uint32_t)bCntW);
    p.dBhw = make_fastdiv((uint32_t)(bCntH * bCntW));
    const uint32_t CH = groups * passes;  // blocks per pooling workgroup: a power of two <= 256 * 8
    const uint32_t nPool = (T + CH - 1) / CH;

    // the compaction relates pooling workgroups to its own 256 blocks, which needs CH to divide 256
    if (CH > 256) return hipErrorInvalidConfiguration;

    hipLaunchKernelGGL(k_reduce_pool, dim3(nPool), dim3(256), 0, stream, mask, p, flags, counts);
    CompactArgs c;
    c.T = T;
    c.nCounts = nPool;
    c.ratio = 256u / CH;
    c.scanned = nPool > SCAN_MIN_COUNTS ? 1 : 0;
    c.bCntH = bCntH; c.bCntW = bCntW;
    c.fixupZero = fixupZero ? 1 : 0;
    c.dBw = p.dBw; c.dBhw = p.dBhw;
    if (c.scanned) hipLaunchKernelGGL(k_reduce_scan, dim3(1), dim3(1024), 0, stream, counts, nPool);
    hipLaunchKernelGGL(k_reduce_compact, dim3((T + 255) / 256), dim3(256), 0, stream, flags, counts, c,
                       activeBlockIndices, binCountDevice, hostSignal, hostSeq);
    return hipGetLastError();
}

}  // namespace sbnet
