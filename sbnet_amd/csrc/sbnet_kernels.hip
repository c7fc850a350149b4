// gfx950 (MI355X, CDNA4, wave64) kernels for reduce_mask, sparse_gather and sparse_scatter.
//
// None of the three ops is a contraction, so there is no MFMA here: they are HBM-bound block
// copies plus one tiny pooling reduction.  What the kernels are built around:
//   * 16-byte (dwordx4) accesses along C on the NHWC side, with 8- and 4-byte variants chosen
//     on the host when C or a base pointer does not allow 16;
//   * for the fused NHWC <-> [blocks, C, R, S] transpose, a tile of Ct channels x P block pixels
//     staged through LDS so that both the NHWC side (runs of Ct floats per pixel) and the planar
//     side (runs of P floats per channel) move in long contiguous pieces; the planar runs start
//     at arbitrary 4-byte alignment (27x27 planes are 729 floats), so every run is split into a
//     scalar head, an aligned dwordx4 body and a scalar tail;
//   * several independent loads in flight per lane before the first use;
//   * no integer division in inner loops (multiply-high reciprocals prepared on the host);
//   * wave64 ballot / popcount for the ordered stream compaction of reduce_mask.
//
// Semantics follow the reference's CPU functors (sbnet_tensorflow/sbnet_ops/reduce_mask.cc:68-96,
// sparse_gather.cc:67-88 and 103-130); each kernel cites the lines it reproduces.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "sbnet_launch.h"

namespace sbnet {

// ---------------------------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------------------------

// Exact unsigned division by a run-time constant: q = (t + ((n - t) >> sh1)) >> sh2 with
// t = mulhi(mul, n).  Valid for every 32-bit n and every d >= 1.
struct FastDiv {
    uint32_t mul, sh1, sh2, d;
};

static FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    uint64_t m = ((1ull << 32) * ((1ull << l) - d)) / d + 1;
    f.mul = (uint32_t)m;
    f.sh1 = l ? 1u : 0u;
    f.sh2 = l ? l - 1u : 0u;
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv& f)
{
    uint32_t t = __umulhi(f.mul, n);
    return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

template <int VEC> struct Vec;
template <> struct Vec<4> { typedef float4 type; };
template <> struct Vec<2> { typedef float2 type; };
template <> struct Vec<1> { typedef float type; };

template <int VEC> __device__ __forceinline__ typename Vec<VEC>::type vzero();
template <> __device__ __forceinline__ float4 vzero<4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <> __device__ __forceinline__ float2 vzero<2>() { return make_float2(0.f, 0.f); }
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }

__device__ __forceinline__ float vget(const float4& v, int k) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; }
__device__ __forceinline__ float vget(const float2& v, int k) { return k == 0 ? v.x : v.y; }
__device__ __forceinline__ float vget(const float& v, int) { return v; }
__device__ __forceinline__ void vset(float4& v, int k, float f) { if (k == 0) v.x = f; else if (k == 1) v.y = f; else if (k == 2) v.z = f; else v.w = f; }
__device__ __forceinline__ void vset(float2& v, int k, float f) { if (k == 0) v.x = f; else v.y = f; }
__device__ __forceinline__ void vset(float& v, int, float f) { v = f; }

__device__ __forceinline__ float4 vadd(const float4& a, const float4& b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
__device__ __forceinline__ float2 vadd(const float2& a, const float2& b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float vadd(const float& a, const float& b) { return a + b; }

// Hardware fp32 atomic add (global_atomic_add_f32, no return value).
__device__ __forceinline__ void atomic_add_f32(float* p, float v) { unsafeAtomicAdd(p, v); }

// Writes one vector of a block into the base tensor: "=", "+=" or atomic "+="
// (sparse_gather.cc:121-128; the atomic flavour is the GPU-only attribute of the op).
template <int VEC, int MODE>
__device__ __forceinline__ void commit(typename Vec<VEC>::type* dst, const typename Vec<VEC>::type& v)
{
    if (MODE == SCATTER_ASSIGN) {
        *dst = v;
    } else if (MODE == SCATTER_ADD) {
        *dst = vadd(*dst, v);
    } else {
        float* d = reinterpret_cast<float*>(dst);
#pragma unroll
        for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v, k));
    }
}

// Reads the (n, bh, bw) triple of block ib (wave-uniform) and derives the block origin.
struct BlockOrigin {
    int n, h0, w0;
    bool valid;  // n inside [0, N): guards against garbage rows in the index list
};

__device__ __forceinline__ BlockOrigin load_origin(const int16_t* __restrict__ idx, uint32_t ib, const Geom& g)
{
    BlockOrigin o;
    const int16_t* t = idx + (size_t)ib * 3;
    o.n = t[0];
    o.h0 = g.oh + (int)t[1] * g.U;
    o.w0 = g.ow + (int)t[2] * g.V;
    o.valid = (unsigned)o.n < (unsigned)g.N;
    return o;
}

// ---------------------------------------------------------------------------------------------
// NHWC block stack <-> NHWC tensor: row-segment copies
// ---------------------------------------------------------------------------------------------
//
// A block in the stack is R rows of rowV = S*C/VEC vectors, contiguous.  The matching piece of
// the tensor is R row segments of the same length (the in-range part of it).  One wave handles
// one "unit": CHUNK = 64*UNR consecutive vectors of one block; four units per workgroup.

constexpr int NHWC_UNR = 8;
constexpr int NHWC_CHUNK = 64 * NHWC_UNR;

struct NhwcArgs {
    Geom g;
    uint32_t rowV;    // vectors per block row, S*C/VEC
    uint32_t blockV;  // vectors per block, R*rowV
    uint32_t cpb;     // chunks per block
    uint32_t units;   // numActive * cpb
    FastDiv dCpb, dRow;
};

// sparse_gather.cc:67-88 with transpose == false.
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_nhwc(const float* __restrict__ x, float* __restrict__ y,
                                                     const int16_t* __restrict__ idx, NhwcArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = load_origin(idx, ib, a.g);
    const int CV = a.g.C / VEC;
    // columns [slo, shi) of the block lie inside the image
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const vec* __restrict__ xv = reinterpret_cast<const vec*>(x);
    vec* __restrict__ yb = reinterpret_cast<vec*>(y) + (size_t)ib * a.blockV;
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;

    vec v[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        v[u] = vzero<VEC>();
        if (e < a.blockV) {
            const uint32_t r = fdiv(e, a.dRow);
            const int j = (int)(e - r * a.rowV);
            const int hh = o.h0 + (int)r;
            if (o.valid && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi) {
                const int64_t src = (((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0) * CV + j;
                v[u] = xv[src];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        if (e < a.blockV) yb[e] = v[u];
    }
}

// sparse_gather.cc:103-130 with transpose == false.
template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_nhwc(const float* __restrict__ x, float* __restrict__ y,
                                                      const int16_t* __restrict__ idx, NhwcArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = load_origin(idx, ib, a.g);
    if (!o.valid) return;
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const vec* __restrict__ xb = reinterpret_cast<const vec*>(x) + (size_t)ib * a.blockV;
    vec* __restrict__ yv = reinterpret_cast<vec*>(y);
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;

    vec v[NHWC_UNR];
    int64_t dst[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        dst[u] = -1;
        v[u] = vzero<VEC>();
        if (e < a.blockV) {
            const uint32_t r = fdiv(e, a.dRow);
            const int j = (int)(e - r * a.rowV);
            const int hh = o.h0 + (int)r;
            if ((unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi) {
                dst[u] = (((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0) * CV + j;
                v[u] = xb[e];
            }
        }
    }
    if (MODE == SCATTER_ADD) {
        vec cur[NHWC_UNR];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) cur[u] = yv[dst[u]];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) yv[dst[u]] = vadd(cur[u], v[u]);
    } else {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) commit<VEC, MODE>(yv + dst[u], v[u]);
    }
}

// ---------------------------------------------------------------------------------------------
// planar block stack [blocks, C, R, S] <-> NHWC tensor: LDS-staged transpose
// ---------------------------------------------------------------------------------------------
//
// One workgroup moves one tile: Ct channels x Pn pixels of one block, where pixels are numbered
// p = r*S + s inside the block.  LDS holds the tile as [Ct][Pp] floats (row pitch Pp >= P, chosen
// so the transposing accesses spread over the banks).  On the NHWC side a lane moves VEC channels
// of one pixel (lanes of a wave cover Ct/VEC consecutive vectors of a pixel, then the next pixel);
// on the planar side a wave moves one channel row of the tile, a contiguous run of Pn floats.
//
// Workgroup ids are remapped so that the tiles of one block (its channel chunks and pixel splits)
// run on the same XCD: hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and
// sibling tiles share cache lines (the 2 halves of a 128-byte line when Ct*4 = 64, the ragged
// ends of planar runs), which only merge in an L2 they have in common.

struct TileArgs {
    Geom g;
    int Ct;         // channels per tile; Ct/VEC is a power of two
    int lppLog;     // log2(Ct/VEC): lanes per pixel on the NHWC side
    int P;          // pixels per tile (the last split of a block may hold fewer)
    int Pp;         // LDS row pitch, floats
    int psplit;     // pixel splits per block
    int cchunks;    // channel chunks per block
    uint32_t tpb;   // tiles per block = psplit * cchunks
    uint32_t total; // numActive * tpb
    uint32_t perXcd;  // ceil(total / 8); grid = 8 * perXcd
    FastDiv dTpb, dCch, dS;
};

constexpr int TILE_UNR = 4;

struct TileId {
    uint32_t ib;
    int c0, ctEff, p0, Pn;
};

__device__ __forceinline__ bool tile_of_workgroup(const TileArgs& a, TileId& t)
{
    const uint32_t bid = blockIdx.x;
    const uint32_t id = (bid & 7u) * a.perXcd + (bid >> 3);
    if (id >= a.total) return false;
    t.ib = fdiv(id, a.dTpb);
    const uint32_t rem = id - t.ib * a.tpb;
    const uint32_t pc = fdiv(rem, a.dCch);
    const uint32_t cc = rem - pc * a.cchunks;
    t.c0 = (int)cc * a.Ct;
    t.ctEff = min(a.Ct, a.g.C - t.c0);
    t.p0 = (int)pc * a.P;
    t.Pn = min(a.P, a.g.R * a.g.S - t.p0);
    return true;
}

// Copies one planar run (n floats) between LDS and global memory with an aligned dwordx4 body.
// TO_GLOBAL: LDS -> global, else global -> LDS.  Called by one full wave.
template <bool TO_GLOBAL>
__device__ __forceinline__ void planar_run(float* __restrict__ gptr, float* __restrict__ lptr, int n, uint32_t lane)
{
    const int mis = (int)((reinterpret_cast<uintptr_t>(gptr) >> 2) & 3);
    const int head = min((4 - mis) & 3, n);
    if ((int)lane < head) {
        if (TO_GLOBAL) gptr[lane] = lptr[lane]; else lptr[lane] = gptr[lane];
    }
    const int nb = (n - head) >> 2;
    for (int v = (int)lane; v < nb; v += 64) {
        const int o = head + 4 * v;
        if (TO_GLOBAL) {
            float4 t = make_float4(lptr[o], lptr[o + 1], lptr[o + 2], lptr[o + 3]);
            *reinterpret_cast<float4*>(gptr + o) = t;
        } else {
            float4 t = *reinterpret_cast<const float4*>(gptr + o);
            lptr[o] = t.x; lptr[o + 1] = t.y; lptr[o + 2] = t.z; lptr[o + 3] = t.w;
        }
    }
    const int t0 = head + 4 * nb;
    if ((int)lane < n - t0) {
        if (TO_GLOBAL) gptr[t0 + lane] = lptr[t0 + lane]; else lptr[t0 + lane] = gptr[t0 + lane];
    }
}

// sparse_gather.cc:67-88 with transpose == true: y[ib, c, r, s] = x[n, h0+r, w0+s, c] or 0.
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_planar(const float* __restrict__ x, float* __restrict__ y,
                                                       const int16_t* __restrict__ idx, TileArgs a)
{
    typedef typename Vec<VEC>::type vec;
    extern __shared__ float lds[];
    TileId t;
    if (!tile_of_workgroup(a, t)) return;
    const BlockOrigin o = load_origin(idx, t.ib, a.g);
    const uint32_t tid = threadIdx.x, nthr = blockDim.x;
    const uint32_t lppMask = (1u << a.lppLog) - 1u;
    const uint32_t items = (uint32_t)t.Pn << a.lppLog;
    const vec* __restrict__ xv = reinterpret_cast<const vec*>(x);
    const int CV = a.g.C / VEC;

    for (uint32_t base = 0; base < items; base += nthr * TILE_UNR) {
        vec v[TILE_UNR];
#pragma unroll
        for (int u = 0; u < TILE_UNR; ++u) {
            const uint32_t i = base + u * nthr + tid;
            v[u] = vzero<VEC>();
            if (i < items) {
                const uint32_t pl = i >> a.lppLog, cl = i & lppMask;
                const uint32_t p = (uint32_t)t.p0 + pl;
                const uint32_t r = fdiv(p, a.dS);
                const int hh = o.h0 + (int)r, ww = o.w0 + (int)(p - r * a.g.S);
                const int c = t.c0 + (int)cl * VEC;
                if (o.valid && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W && c < a.g.C)
                    v[u] = xv[(((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * CV + (c / VEC)];
            }
        }
#pragma unroll
        for (int u = 0; u < TILE_UNR; ++u) {
            const uint32_t i = base + u * nthr + tid;
            if (i < items) {
                const uint32_t pl = i >> a.lppLog, cl = i & lppMask;
#pragma unroll
                for (int k = 0; k < VEC; ++k) lds[(cl * VEC + k) * a.Pp + pl] = vget(v[u], k);
            }
        }
    }
    __syncthreads();

    const uint32_t lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
    const int64_t RS = (int64_t)a.g.R * a.g.S;
    for (int c = (int)wave; c < t.ctEff; c += (int)nwaves) {
        float* dst = y + ((int64_t)t.ib * a.g.C + t.c0 + c) * RS + t.p0;
        planar_run<true>(dst, lds + c * a.Pp, t.Pn, lane);
    }
}

// sparse_gather.cc:103-130 with transpose == true: the block stack is [blocks, C, R, S].
template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_planar(const float* __restrict__ x, float* __restrict__ y,
                                                        const int16_t* __restrict__ idx, TileArgs a)
{
    typedef typename Vec<VEC>::type vec;
    extern __shared__ float lds[];
    TileId t;
    if (!tile_of_workgroup(a, t)) return;
    const BlockOrigin o = load_origin(idx, t.ib, a.g);
    if (!o.valid) return;
    const uint32_t tid = threadIdx.x, nthr = blockDim.x;
    const uint32_t lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
    const int64_t RS = (int64_t)a.g.R * a.g.S;

    for (int c = (int)wave; c < t.ctEff; c += (int)nwaves) {
        const float* src = x + ((int64_t)t.ib * a.g.C + t.c0 + c) * RS + t.p0;
        planar_run<false>(const_cast<float*>(src), lds + c * a.Pp, t.Pn, lane);
    }
    __syncthreads();

    const uint32_t lppMask = (1u << a.lppLog) - 1u;
    const uint32_t items = (uint32_t)t.Pn << a.lppLog;
    vec* __restrict__ yv = reinterpret_cast<vec*>(y);
    const int CV = a.g.C / VEC;

    for (uint32_t base = 0; base < items; base += nthr * TILE_UNR) {
        vec v[TILE_UNR];
        int64_t dst[TILE_UNR];
#pragma unroll
        for (int u = 0; u < TILE_UNR; ++u) {
            const uint32_t i = base + u * nthr + tid;
            dst[u] = -1;
            v[u] = vzero<VEC>();
            if (i < items) {
                const uint32_t pl = i >> a.lppLog, cl = i & lppMask;
                const uint32_t p = (uint32_t)t.p0 + pl;
                const uint32_t r = fdiv(p, a.dS);
                const int hh = o.h0 + (int)r, ww = o.w0 + (int)(p - r * a.g.S);
                const int c = t.c0 + (int)cl * VEC;
                if ((unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W && c < a.g.C) {
                    dst[u] = (((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * CV + (c / VEC);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) vset(v[u], k, lds[(cl * VEC + k) * a.Pp + pl]);
                }
            }
        }
        if (MODE == SCATTER_ADD) {
            vec cur[TILE_UNR];
#pragma unroll
            for (int u = 0; u < TILE_UNR; ++u)
                if (dst[u] >= 0) cur[u] = yv[dst[u]];
#pragma unroll
            for (int u = 0; u < TILE_UNR; ++u)
                if (dst[u] >= 0) yv[dst[u]] = vadd(cur[u], v[u]);
        } else {
#pragma unroll
            for (int u = 0; u < TILE_UNR; ++u)
                if (dst[u] >= 0) commit<VEC, MODE>(yv + dst[u], v[u]);
        }
    }
}

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
// the offset of the workgroup.  Triples therefore land in the CPU functor's order, and the last
// workgroup knows the total: it stores the count and applies the "no active block" fix-up
// (reduce_mask.cc:206-218) on the device.
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
    int logG, logGw;  // lanes per block, lanes along w inside a group
    int passes;       // blocks per group
    FastDiv dBw, dBhw;
};

__device__ __forceinline__ float next_down(float f)
{
    if (!(f == f) || f == -INFINITY) return f;
    if (f == 0.f) return -1.401298464e-45f;
    int i = __float_as_int(f);
    i += (f > 0.f) ? -1 : 1;
    return __int_as_float(i);
}

__device__ __forceinline__ float next_up(float f) { return -next_down(-f); }

__global__ __launch_bounds__(256) void k_reduce_pool(const float* __restrict__ mask, PoolArgs a,
                                                     uint8_t* __restrict__ flags, int32_t* __restrict__ counts)
{
    __shared__ int wgCount;
    const uint32_t tid = threadIdx.x;
    if (tid == 0) wgCount = 0;
    __syncthreads();

    const int G = 1 << a.logG, Gw = 1 << a.logGw, Gh = G >> a.logGw;
    const uint32_t groups = 256u >> a.logG;
    const uint32_t grp = tid >> a.logG;
    const int l = (int)(tid & (uint32_t)(G - 1));
    const int lc = l & (Gw - 1), lr = l >> a.logGw;
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
        for (int hh = hlo + lr; hh < hhi; hh += Gh) {
            const float* __restrict__ row = img + (int64_t)hh * a.W;
            for (int ww = wlo + lc; ww < whi; ww += Gw) {
                const float v = row[ww];
                if (a.avg) {
                    sum += v;
                    sabs += fabsf(v);
                    allint &= (v == truncf(v));
                } else {
                    any |= (v > a.tol);
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

struct CompactArgs {
    uint32_t T;
    uint32_t nCounts;   // workgroups of kernel 1
    uint32_t ratio;     // kernel-1 workgroups per 256 blocks
    int bCntH, bCntW;
    int fixupZero;
    FastDiv dBw, dBhw;
};

__global__ __launch_bounds__(256) void k_reduce_compact(const uint8_t* __restrict__ flags,
                                                        const int32_t* __restrict__ counts, CompactArgs a,
                                                        int16_t* __restrict__ idx, int32_t* __restrict__ binCount)
{
    __shared__ int waveSum[4];
    __shared__ int waveCnt[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // active blocks before this workgroup's 256 blocks
    uint32_t nPrev = blockIdx.x * a.ratio;
    if (nPrev > a.nCounts) nPrev = a.nCounts;
    int part = 0;
    for (uint32_t i = tid; i < nPrev; i += 256) part += counts[i];
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
    if (blockIdx.x == gridDim.x - 1 && tid == 0) {
        int total = base + waveCnt[0] + waveCnt[1] + waveCnt[2] + waveCnt[3];
        if (total == 0 && a.fixupZero) {
            idx[0] = 0; idx[1] = 0; idx[2] = 0;
            total = 1;
        }
        *binCount = total;
    }
}

// ---------------------------------------------------------------------------------------------
// flat copy (CopyTensorFunctor, sparse_gather.cc:135-142 / sparse_gather.cu:268-276)
// ---------------------------------------------------------------------------------------------

constexpr int COPY_UNR = 8;

__global__ __launch_bounds__(256) void k_copy_v4(const float4* __restrict__ src, float4* __restrict__ dst, size_t n4)
{
    const size_t base = (size_t)blockIdx.x * (256 * COPY_UNR) + threadIdx.x;
    float4 v[COPY_UNR];
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < n4) v[u] = src[i];
    }
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        if (i < n4) dst[i] = v[u];
    }
}

__global__ __launch_bounds__(256) void k_copy_scalar(const float* __restrict__ src, float* __restrict__ dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

// ---------------------------------------------------------------------------------------------
// host side: launch configuration
// ---------------------------------------------------------------------------------------------

static int ilog2_floor(uint32_t v)
{
    int l = 0;
    while ((2u << l) <= v) ++l;
    return l;
}

static uint32_t pow2_ceil(uint32_t v)
{
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

// Optional overrides for experiments: SBNET_TUNE="ct=32,lds=49152,wg=256".
struct Tune {
    int ct = 0, ldsBytes = 0, wg = 0;
};

static Tune read_tune()
{
    Tune t;
    const char* s = getenv("SBNET_TUNE");
    if (!s) return t;
    const char* p;
    if ((p = strstr(s, "ct="))) t.ct = atoi(p + 3);
    if ((p = strstr(s, "lds="))) t.ldsBytes = atoi(p + 4);
    if ((p = strstr(s, "wg="))) t.wg = atoi(p + 3);
    return t;
}

static int pick_vec(const Geom& g, const void* a, const void* b)
{
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
    if (g.C % 4 == 0 && (bits & 15) == 0) return 4;
    if (g.C % 2 == 0 && (bits & 7) == 0) return 2;
    return 1;
}

size_t reduce_mask_workspace_bytes(int64_t totalBlocks)
{
    // flag bytes (padded to 16) + worst-case one count per block + the total
    const size_t flags = ((size_t)totalBlocks + 15) & ~(size_t)15;
    return flags + (size_t)totalBlocks * sizeof(int32_t) + 16;
}

hipError_t launch_reduce_mask(const float* mask, const Geom& g, int bCntH, int bCntW, float tol,
                              bool avgPool, bool fixupZero, int16_t* activeBlockIndices,
                              int32_t* binCountDevice, void* workspace, hipStream_t stream)
{
    const uint32_t T = (uint32_t)((int64_t)g.N * bCntH * bCntW);
    uint8_t* flags = static_cast<uint8_t*>(workspace);
    const size_t flagBytes = ((size_t)T + 15) & ~(size_t)15;
    int32_t* counts = reinterpret_cast<int32_t*>(flags + flagBytes);
    if (!binCountDevice) binCountDevice = counts + T;

    PoolArgs p;
    p.N = g.N; p.H = g.H; p.W = g.W;
    p.R = g.R; p.S = g.S; p.U = g.U; p.V = g.V; p.oh = g.oh; p.ow = g.ow;
    p.bCntH = bCntH; p.bCntW = bCntW;
    p.T = T;
    p.tol = tol;
    p.avg = avgPool ? 1 : 0;
    const uint64_t npx = (uint64_t)g.R * (uint64_t)g.S;
    int logG = npx >= 16 ? ilog2_floor((uint32_t)(npx / 8 > 64 ? 64 : npx / 8)) : 0;
    if (logG > 6) logG = 6;
    p.logG = logG;
    const uint32_t Gw = pow2_ceil((uint32_t)g.S);
    p.logGw = ilog2_floor(Gw < (1u << logG) ? Gw : (1u << logG));
    const uint32_t groups = 256u >> logG;
    int passes = 1;
    while (passes < (1 << logG) && passes < 8 && T / (groups * passes) > 2048) passes *= 2;
    p.passes = passes;
    p.dBw = make_fastdiv((uint32_t)bCntW);
    p.dBhw = make_fastdiv((uint32_t)(bCntH * bCntW));
    const uint32_t CH = groups * passes;  // a power of two <= 256 * 8
    const uint32_t nPool = (T + CH - 1) / CH;

    // kernel 2 sums the counts of the pooling workgroups that lie wholly before its 256 blocks,
    // which needs CH to divide 256
    if (CH > 256) return hipErrorInvalidConfiguration;

    hipLaunchKernelGGL(k_reduce_pool, dim3(nPool), dim3(256), 0, stream, mask, p, flags, counts);

    CompactArgs c;
    c.T = T;
    c.nCounts = nPool;
    c.ratio = 256u / CH;
    c.bCntH = bCntH; c.bCntW = bCntW;
    c.fixupZero = fixupZero ? 1 : 0;
    c.dBw = p.dBw; c.dBhw = p.dBhw;
    hipLaunchKernelGGL(k_reduce_compact, dim3((T + 255) / 256), dim3(256), 0, stream, flags, counts, c,
                       activeBlockIndices, binCountDevice);
    return hipGetLastError();
}

static bool make_nhwc_args(const Geom& g, int numActive, int vec, NhwcArgs& a)
{
    a.g = g;
    const uint64_t rowV = (uint64_t)g.S * g.C / vec;
    const uint64_t blockV = rowV * g.R;
    if (blockV >= (1ull << 31)) return false;
    a.rowV = (uint32_t)rowV;
    a.blockV = (uint32_t)blockV;
    a.cpb = (uint32_t)((blockV + NHWC_CHUNK - 1) / NHWC_CHUNK);
    const uint64_t units = (uint64_t)numActive * a.cpb;
    if (units >= (1ull << 31)) return false;
    a.units = (uint32_t)units;
    a.dCpb = make_fastdiv(a.cpb);
    a.dRow = make_fastdiv(a.rowV);
    return true;
}

// Chooses the LDS tile of the planar kernels.
static bool make_tile_args(const Geom& g, int numActive, int vec, TileArgs& a, int& threads, size_t& ldsBytes)
{
    static const Tune tune = read_tune();
    a.g = g;
    const int64_t RS64 = (int64_t)g.R * g.S;
    if (RS64 >= (1ll << 30)) return false;
    const int RS = (int)RS64;
    // channels per tile: 32 floats (one 128-byte line per pixel) unless C is smaller
    int ctWant = tune.ct > 0 ? tune.ct : 32;
    int lpp = 1;
    while (lpp * 2 * vec <= ctWant && lpp * vec < g.C) lpp *= 2;
    a.Ct = lpp * vec;
    a.lppLog = ilog2_floor((uint32_t)lpp);
    a.cchunks = (g.C + a.Ct - 1) / a.Ct;
    // pixels per tile: keep a tile within the LDS budget so several workgroups share a CU
    const int budget = tune.ldsBytes > 0 ? tune.ldsBytes : 40 * 1024;
    int maxP = budget / (a.Ct * 4) - 16;
    if (maxP < 16) maxP = 16;
    a.psplit = (RS + maxP - 1) / maxP;
    a.P = (RS + a.psplit - 1) / a.psplit;
    a.psplit = (RS + a.P - 1) / a.P;
    // pitch: vec*Pp == 64/lpp (mod 64) makes a wave's transposing LDS accesses hit 64 distinct banks
    int Pp = a.P;
    if (lpp * vec <= 64) {
        const int want = (64 / lpp) % 64;
        while ((vec * Pp) % 64 != want) ++Pp;
    } else {
        Pp |= 1;
    }
    a.Pp = Pp;
    a.tpb = (uint32_t)(a.psplit * a.cchunks);
    const uint64_t total = (uint64_t)numActive * a.tpb;
    if (total >= (1ull << 31) - 8) return false;
    a.total = (uint32_t)total;
    a.perXcd = (a.total + 7) / 8;
    a.dTpb = make_fastdiv(a.tpb);
    a.dCch = make_fastdiv((uint32_t)a.cchunks);
    a.dS = make_fastdiv((uint32_t)g.S);
    ldsBytes = (size_t)a.Ct * a.Pp * sizeof(float);
    const int elems = a.Ct * a.P;
    threads = tune.wg > 0 ? tune.wg : (elems >= 4096 ? 256 : elems >= 1536 ? 128 : 64);
    return ldsBytes <= 64 * 1024;
}

template <int VEC>
static void gather_dispatch(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive,
                            bool transpose, hipStream_t stream, hipError_t& err)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        hipLaunchKernelGGL(k_gather_nhwc<VEC>, dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        if (!make_tile_args(g, numActive, VEC, a, threads, lds)) { err = hipErrorInvalidValue; return; }
        hipLaunchKernelGGL(k_gather_planar<VEC>, dim3(a.perXcd * 8), dim3(threads), lds, stream, x, y, idx, a);
    }
}

hipError_t launch_gather(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                         bool transpose, hipStream_t stream)
{
    if (numActive == 0) return hipSuccess;
    hipError_t err = hipSuccess;
    // the planar side of the transpose handles its own alignment; only the NHWC pointer matters there
    const int vec = pick_vec(g, x, transpose ? nullptr : y);
    if (vec == 4) gather_dispatch<4>(x, y, idx, g, numActive, transpose, stream, err);
    else if (vec == 2) gather_dispatch<2>(x, y, idx, g, numActive, transpose, stream, err);
    else gather_dispatch<1>(x, y, idx, g, numActive, transpose, stream, err);
    if (err != hipSuccess) return err;
    return hipGetLastError();
}

template <int VEC, int MODE>
static void scatter_dispatch(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive,
                             bool transpose, hipStream_t stream, hipError_t& err)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        hipLaunchKernelGGL((k_scatter_nhwc<VEC, MODE>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        if (!make_tile_args(g, numActive, VEC, a, threads, lds)) { err = hipErrorInvalidValue; return; }
        hipLaunchKernelGGL((k_scatter_planar<VEC, MODE>), dim3(a.perXcd * 8), dim3(threads), lds, stream, x, y, idx, a);
    }
}

template <int VEC>
static void scatter_mode(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive,
                         bool transpose, ScatterMode mode, hipStream_t stream, hipError_t& err)
{
    if (mode == SCATTER_ASSIGN) scatter_dispatch<VEC, SCATTER_ASSIGN>(x, y, idx, g, numActive, transpose, stream, err);
    else if (mode == SCATTER_ADD) scatter_dispatch<VEC, SCATTER_ADD>(x, y, idx, g, numActive, transpose, stream, err);
    else scatter_dispatch<VEC, SCATTER_ATOMIC>(x, y, idx, g, numActive, transpose, stream, err);
}

hipError_t launch_scatter(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                          bool transpose, ScatterMode mode, hipStream_t stream)
{
    if (numActive == 0) return hipSuccess;
    hipError_t err = hipSuccess;
    const int vec = pick_vec(g, y, transpose ? nullptr : x);
    if (vec == 4) scatter_mode<4>(x, y, idx, g, numActive, transpose, mode, stream, err);
    else if (vec == 2) scatter_mode<2>(x, y, idx, g, numActive, transpose, mode, stream, err);
    else scatter_mode<1>(x, y, idx, g, numActive, transpose, mode, stream, err);
    if (err != hipSuccess) return err;
    return hipGetLastError();
}

hipError_t launch_copy(float* dst, const float* src, size_t count, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
    if ((bits & 15) == 0) {
        const size_t n4 = count / 4;
        if (n4) {
            const size_t per = 256 * COPY_UNR;
            hipLaunchKernelGGL(k_copy_v4, dim3((unsigned)((n4 + per - 1) / per)), dim3(256), 0, stream,
                               reinterpret_cast<const float4*>(src), reinterpret_cast<float4*>(dst), n4);
        }
        const size_t rem = count - n4 * 4;
        if (rem) hipLaunchKernelGGL(k_copy_scalar, dim3(1), dim3(256), 0, stream, src + n4 * 4, dst + n4 * 4, rem);
    } else {
        size_t wgs = (count + 255) / 256;
        if (wgs > 65536) wgs = 65536;
        hipLaunchKernelGGL(k_copy_scalar, dim3((unsigned)wgs), dim3(256), 0, stream, src, dst, count);
    }
    return hipGetLastError();
}

}  // namespace sbnet
