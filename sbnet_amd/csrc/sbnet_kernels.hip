// gfx950 (MI355X, CDNA4, wave64) kernels for reduce_mask, sparse_gather and sparse_scatter.
//
// None of the three ops is a contraction, so there is no MFMA here: they are HBM-bound block
// copies plus one tiny pooling reduction.  What the kernels are built around:
//   * 16-byte (dwordx4) accesses along C on the NHWC side, with 8- and 4-byte variants chosen
//     on the host when C or a base pointer does not allow 16;
//   * for the fused NHWC <-> [blocks, C, R, S] transpose, a tile of Ct channels x P block pixels
//     staged through LDS so that both the NHWC side (runs of Ct floats per pixel) and the planar
//     side (runs of P floats per channel) move in long contiguous pieces; the planar runs start
//     at arbitrary 4-byte alignment (27x27 planes are 729 floats): the scatter reads them as
//     misaligned dwordx4 slots, the gather writes whole, aligned 128-byte lines;
//   * raw buffer addressing with out-of-range offsets instead of branches around loads and stores;
//   * several independent loads in flight per lane before the first use;
//   * no integer division in inner loops (multiply-high reciprocals prepared on the host);
//   * wave64 ballot / popcount for the ordered stream compaction of reduce_mask.
//
// Semantics follow the reference's CPU functors (sbnet_tensorflow/sbnet_ops/reduce_mask.cc:68-96,
// sparse_gather.cc:67-88 and 103-130); each kernel cites the lines it reproduces.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

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

// Native clang vectors (not HIP's float4 struct): they take the nontemporal builtins and arithmetic.
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

template <int VEC> struct Vec;
template <> struct Vec<4> { typedef f4 type; };
template <> struct Vec<2> { typedef f2 type; };
template <> struct Vec<1> { typedef float type; };

template <int VEC> __device__ __forceinline__ typename Vec<VEC>::type vzero();
template <> __device__ __forceinline__ f4 vzero<4>() { return (f4)(0.f); }
template <> __device__ __forceinline__ f2 vzero<2>() { return (f2)(0.f); }
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }

__device__ __forceinline__ float vget(const f4& v, int k) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; }
__device__ __forceinline__ float vget(const f2& v, int k) { return k == 0 ? v.x : v.y; }
__device__ __forceinline__ float vget(const float& v, int) { return v; }
__device__ __forceinline__ void vset(f4& v, int k, float f) { if (k == 0) v.x = f; else if (k == 1) v.y = f; else if (k == 2) v.z = f; else v.w = f; }
__device__ __forceinline__ void vset(f2& v, int k, float f) { if (k == 0) v.x = f; else v.y = f; }
__device__ __forceinline__ void vset(float& v, int, float f) { v = f; }

template <typename T> __device__ __forceinline__ T vadd(const T& a, const T& b) { return a + b; }

// Streaming accesses: every byte of x, of the block stack and of the base tensor is touched once per
// op, so loads and stores carry the nontemporal hint (measured: a plain dwordx4 copy gains ~10 %).
template <typename T> __device__ __forceinline__ T ld_stream(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void st_stream(T* p, const T& v) { __builtin_nontemporal_store(v, p); }

// Hardware fp32 atomic add (global_atomic_add_f32, no return value).
__device__ __forceinline__ void atomic_add_f32(float* p, float v) { unsafeAtomicAdd(p, v); }

// Writes one vector of a block into the base tensor: "=", "+=" or atomic "+="
// (sparse_gather.cc:121-128; the atomic flavour is the GPU-only attribute of the op).
template <int VEC, int MODE>
__device__ __forceinline__ void commit(typename Vec<VEC>::type* dst, const typename Vec<VEC>::type& v)
{
    if (MODE == SCATTER_ASSIGN) {
        st_stream(dst, v);
    } else if (MODE == SCATTER_ADD) {
        st_stream(dst, vadd(ld_stream(dst), v));
    } else {
        float* d = reinterpret_cast<float*>(dst);
#pragma unroll
        for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v, k));
    }
}

// Reads the (n, bh, bw) triple of block ib (wave-uniform) and derives the block origin.
struct BlockOrigin {
    int n, h0, w0;
    int bh, bw;  // the block's grid position
    bool valid;  // n inside [0, N): guards against garbage rows in the index list
};

__device__ __forceinline__ BlockOrigin load_origin(const int16_t* __restrict__ idx, uint32_t ib, const Geom& g)
{
    BlockOrigin o;
    const int16_t* t = idx + (size_t)ib * 3;
    o.n = t[0];
    o.bh = t[1];
    o.bw = t[2];
    o.h0 = g.oh + o.bh * g.U;
    o.w0 = g.ow + o.bw * g.V;
    o.valid = (unsigned)o.n < (unsigned)g.N;
    return o;
}

// The same in two steps, for software pipelines: the loads are issued early and the arithmetic (which
// is what makes a wave wait for them) happens where the origin is first needed.
struct RawTriple {
    uint32_t lo, hi;  // the two aligned dwords that hold the 6-byte triple
    uint32_t shift;   // 0 or 16: where the triple starts inside them
};

// ib is the same for the whole workgroup.  Reading the two aligned dwords around the triple from a uniform
// address lets the compiler use the scalar unit, whose loads are counted apart from vector loads and stores:
// waiting for the triple then does not wait for the stores in flight.  (A triple that ends the list on a
// 4-byte boundary + 2 makes the second dword reach 2 bytes past the list, inside the same aligned dword.)
__device__ __forceinline__ RawTriple load_triple(const int16_t* __restrict__ idx, uint32_t ib)
{
    const uint32_t byteOff = 6u * (uint32_t)__builtin_amdgcn_readfirstlane(ib);
    const uintptr_t base = reinterpret_cast<uintptr_t>(idx) + byteOff;
    // constant address space: a uniform address alone does not make the compiler pick a scalar load, and a
    // triple that arrives in vector registers makes every descriptor built from it "divergent" (each buffer
    // access then sits in a readfirstlane loop).  The list is never written by the kernels that read it.
    typedef const uint32_t __attribute__((address_space(4))) * const_u32_ptr;
    const_u32_ptr w = (const_u32_ptr)(base & ~(uintptr_t)3);
    RawTriple r;
    r.lo = w[0];
    r.hi = w[1];
    r.shift = (uint32_t)(base & 2) * 8u;
    return r;
}

__device__ __forceinline__ BlockOrigin origin_of(const RawTriple& r, const Geom& g)
{
    const uint64_t bits = (((uint64_t)r.hi << 32) | r.lo) >> r.shift;
    BlockOrigin o;
    o.n = (int)(int16_t)(bits & 0xffffu);
    o.bh = (int)(int16_t)((bits >> 16) & 0xffffu);
    o.bw = (int)(int16_t)((bits >> 32) & 0xffffu);
    o.h0 = g.oh + o.bh * g.U;
    o.w0 = g.ow + o.bw * g.V;
    o.valid = (unsigned)o.n < (unsigned)g.N;
    return o;
}

// True for list rows at or beyond the device-resident count (see Geom::countDev); ib is wave-uniform.
__device__ __forceinline__ bool beyond_count(const Geom& g, uint32_t ib)
{
    if (!g.countDev) return false;
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    return ib >= (uint32_t)*(const_i32_ptr)(reinterpret_cast<uintptr_t>(g.countDev));
}

// Overlapping scatter-add in passes ("colours").  Blocks whose grid positions agree modulo
// (Kh, Kw) = (ceil(R/U), ceil(S/V)) cannot overlap, so a launch that handles one residue class can add
// with plain load-add-store; Kh*Kw launches in a row cover the list.  The result is reproducible (the
// order of the adds is the order of the passes) and runs at streaming speed, where hardware atomics reach
// about a tenth of it.  A block listed twice breaks the premise: the map kernel of the pull scatter
// detects that (`dup`), and then pass 0 handles every block with atomics and the other passes do nothing.
constexpr int SCATTER_COLOR = 3;  // kernel-side mode; callers ask for SCATTER_ATOMIC

// Plain writes ("=") of overlapping blocks in the sequential CPU functor's order: that functor visits the
// list front to back (sparse_gather.cc:105), so on a pixel that several blocks cover the one listed last
// wins.  A per-pixel owner map (the highest list position that covers the pixel, built by k_owner_fill and
// k_owner_mark before the launch) lets every block write only the pixels it owns: no pixel is written twice,
// and a block listed twice is handled like any other overlap.
constexpr int SCATTER_OWNED = 4;  // kernel-side mode; callers ask for SCATTER_ASSIGN and give scratch

// The same order without a per-pixel map, for the common case of at most 2x2 blocks over a pixel (bsize <= 2 *
// bstride) and a list short enough to compare every pair of blocks: a block's eight grid neighbours (and any other
// row of the list that names the block itself) are the only blocks that can share pixels with it, and which of
// its pixels a neighbour covers depends only on whether the pixel lies in the block's first R - U rows (shared
// with the row of blocks above), its rows from U on (shared with the row below), or in between, and likewise for
// columns.  k_rank_table leaves nine bits per block: bit 3*rowClass + colClass is set when some block listed
// later covers that class of pixels; the scatter kernels skip those pixels.
constexpr int SCATTER_RANKED = 5;  // kernel-side mode; callers ask for SCATTER_ASSIGN and give scratch

struct ColorArgs {
    int kh, kw, pass;
    const int32_t* dup;
    const int32_t* owner;  // SCATTER_OWNED: [N, H, W] list positions, -1 where no block covers the pixel
    const int32_t* rank;   // SCATTER_RANKED: nine bits per block, see k_rank_table
};

// Pixel (r, s) of a block against the block's nine bits: true when a block listed later covers it.
__device__ __forceinline__ bool ranked_out(uint32_t bits, uint32_t r, uint32_t s, const Geom& g)
{
    const uint32_t rc = (int)r < g.R - g.U ? 0u : ((int)r >= g.U ? 2u : 1u);
    const uint32_t cc = (int)s < g.S - g.V ? 0u : ((int)s >= g.V ? 2u : 1u);
    return (bits >> (rc * 3u + cc)) & 1u;
}

__device__ __forceinline__ uint32_t rank_bits(const ColorArgs& col, uint32_t ib)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;  // ib is wave-uniform: scalar load
    return (uint32_t)*(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.rank + ib));
}

// True when this launch has nothing to do for the block; `atomics` tells how to add otherwise.
__device__ __forceinline__ bool color_skip(const ColorArgs& col, const BlockOrigin& o, bool& atomics)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    atomics = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.dup)) != 0;  // written by an earlier kernel
    if (atomics) return col.pass != 0;
    int mh = o.bh % col.kh, mw = o.bw % col.kw;
    if (mh < 0) mh += col.kh;
    if (mw < 0) mw += col.kw;
    return mh * col.kw + mw != col.pass;
}

// ---------------------------------------------------------------------------------------------
// NHWC block stack <-> NHWC tensor: row-segment copies
// ---------------------------------------------------------------------------------------------
//
// A block in the stack is R rows of rowV = S*C/VEC vectors, contiguous.  The matching piece of
// the tensor is R row segments of the same length (the in-range part of it).  One wave handles
// one "unit": CHUNK = 64*UNR consecutive vectors of one block; four units per workgroup.

constexpr int NHWC_UNR = 4;  // 4 KB per wave, 16 KB per workgroup (see COPY_UNR)
constexpr int NHWC_CHUNK = 64 * NHWC_UNR;

struct NhwcArgs {
    Geom g;
    uint32_t rowV;    // vectors per block row, S*C/VEC
    uint32_t blockV;  // vectors per block, R*rowV
    uint32_t cpb;     // chunks per block
    uint32_t units;   // numActive * cpb
    FastDiv dCpb, dRow, dCV;  // dCV: by the vectors per pixel, C/VEC
};

// sparse_gather.cc:67-88 with transpose == false.
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_nhwc_wide(const float* __restrict__ x, float* __restrict__ y,
                                                     const int16_t* __restrict__ idx, NhwcArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);  // ib is wave-uniform: scalar load
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
                v[u] = ld_stream(xv + src);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        if (e < a.blockV) st_stream(yb + e, v[u]);
    }
}

// sparse_gather.cc:103-130 with transpose == false.
template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_nhwc_wide(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, NhwcArgs a, ColorArgs col)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);  // ib is wave-uniform: scalar load
    if (!o.valid) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, o, atomics)) return;
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const vec* __restrict__ xb = reinterpret_cast<const vec*>(x) + (size_t)ib * a.blockV;
    vec* yv = reinterpret_cast<vec*>(y);
    const vec* ysv = reinterpret_cast<const vec*>(ysrc);  // what an add reads: y itself, or the base y is a copy of
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
                if (MODE == SCATTER_OWNED &&
                    col.owner[((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0 + (int)fdiv((uint32_t)j, a.dCV)] != (int32_t)ib)
                    dst[u] = -1;
                else if (MODE == SCATTER_RANKED && ranked_out(rank_bits(col, ib), r, fdiv((uint32_t)j, a.dCV), a.g))
                    dst[u] = -1;
                else
                    v[u] = ld_stream(xb + e);
            }
        }
    }
    if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
        vec cur[NHWC_UNR];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) cur[u] = ld_stream(ysv + dst[u]);
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) st_stream(yv + dst[u], vadd(cur[u], v[u]));
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_OWNED || MODE == SCATTER_RANKED) {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) commit<VEC, SCATTER_ASSIGN>(yv + dst[u], v[u]);
    } else {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) commit<VEC, SCATTER_ATOMIC>(yv + dst[u], v[u]);
    }
}

// ---------------------------------------------------------------------------------------------
// planar block stack [blocks, C, R, S] <-> NHWC tensor: LDS-staged transpose
// ---------------------------------------------------------------------------------------------
//
// A tile is Ct channels x Pn pixels of one block, pixels numbered p = r*S + s inside the block.
// On the NHWC side a lane moves VEC channels of one pixel (the lanes of a wave cover the Ct/VEC
// vectors of a pixel, then the next pixel).  On the planar side row c of the tile is a contiguous
// run of Pn floats that starts at whatever 4-byte alignment (c*R*S + p0) lands on (27x27 planes hold
// 729 floats).  Runs move as dwordx4 "slots" of 4 consecutive floats from the start of the run, so
// most of these accesses are not 16-byte aligned; gfx950 executes misaligned global dwordx4 accesses
// at the speed of aligned ones (measured with a plain copy), which makes an aligned-body / scalar-
// head-and-tail split unnecessary.  Only the last slot of a run can be partial.
//
// One workgroup moves one tile: all of its global loads are issued back to back into registers (no
// control flow around them: lanes with nothing to fetch use an out-of-range buffer offset, which reads
// as zero), then go through LDS, then leave as stores.  A persistent variant that
// software-pipelined several tiles per workgroup (loads of tile i+1 in flight during the stores of tile
// i) was measured slower the more tiles a workgroup owned (47 -> 52 -> 65 us for 1, 4, 12 tiles per
// workgroup on the 800x800x128 workload): the hardware dispatcher balances one-tile workgroups better
// than a static split, and with 4-5 workgroups resident per CU their phases overlap anyway.  Tiles are
// numbered (block, channel chunk, pixel split) with the pixel split fastest, so the splits of one
// channel chunk, which continue each other's planar runs, are dispatched together.
//
// LDS layout: tile row c at c*Pp floats, Pp a multiple of 32, pixel e at column e.  Columns are
// XOR-swizzled in units of 4 floats by ((c >> 2) & 7): the planar side still sees aligned groups of
// 4 floats (ds_read_b128 / ds_write_b128), and the transposing NHWC side, where 32 lanes touch 4
// consecutive pixels of 8 different channel groups at once, hits 32 distinct banks (LDS has 32
// four-byte banks; a padded, unswizzled layout lost 58 % of its LDS cycles to bank conflicts).

constexpr int TILE_LD = 4;  // vectors (NHWC side) or slots (planar side) held in registers per thread

struct TileArgs {
    Geom g;
    int Ct;             // channels per tile; Ct/VEC is a power of two
    int lppLog;         // log2(Ct/VEC): lanes per pixel on the NHWC side
    int P;              // pixels per tile (the last split of a block may hold fewer)
    int Pp;             // LDS row pitch in floats, multiple of 32, >= P
    int psplit;         // pixel splits per block
    int cchunks;        // channel chunks per block
    uint32_t tpb;       // tiles per block = psplit * cchunks
    uint32_t total;     // numActive * tpb
    int grid2d;         // the launch is (tpb, block rows): see for_each_block_of_workgroup
    uint32_t blocks;    // capacity of the block list (numActive)
    uint32_t vpr;       // slots per planar row: (P + 3) / 4
    int64_t imgFloats;  // H * W * C
    uint32_t imgBytes;  // H * W * C * 4, below 2^32 (the host falls back to k_planar_small otherwise)
    FastDiv dTpb, dPs, dS, dVpr;
};

struct TileId {
    uint32_t ib;
    int c0, ctEff, p0, Pn;
};

// Geometry of a tile launch: read from the argument struct, or fixed at compile time (see LinesRt / LinesFixed
// further down for what that buys).
struct TileRt {
    static constexpr bool FIXED = false;
    __device__ static uint32_t nthr(const TileArgs&) { return blockDim.x; }
    __device__ static uint32_t S(const TileArgs& a) { return (uint32_t)a.g.S; }
    __device__ static uint32_t C(const TileArgs& a) { return (uint32_t)a.g.C; }
    __device__ static uint32_t RS(const TileArgs& a) { return (uint32_t)(a.g.R * a.g.S); }
    __device__ static uint32_t P(const TileArgs& a) { return (uint32_t)a.P; }
    __device__ static uint32_t Pp(const TileArgs& a) { return (uint32_t)a.Pp; }
    __device__ static uint32_t psplit(const TileArgs& a) { return (uint32_t)a.psplit; }
    __device__ static uint32_t Ct(const TileArgs& a) { return (uint32_t)a.Ct; }
    __device__ static uint32_t lppLog(const TileArgs& a) { return (uint32_t)a.lppLog; }
    __device__ static uint32_t tpb(const TileArgs& a) { return a.tpb; }
    __device__ static uint32_t vpr(const TileArgs& a) { return a.vpr; }
    __device__ static uint32_t divS(uint32_t v, const TileArgs& a) { return fdiv(v, a.dS); }
    __device__ static uint32_t divPs(uint32_t v, const TileArgs& a) { return fdiv(v, a.dPs); }
    __device__ static uint32_t divTpb(uint32_t v, const TileArgs& a) { return fdiv(v, a.dTpb); }
    __device__ static uint32_t divVpr(uint32_t v, const TileArgs& a) { return fdiv(v, a.dVpr); }
};

// 4-float channel vectors only (C_ a multiple of 4); P_ pixels per tile.
template <int R_, int S_, int C_, int P_, int NTHR_>
struct TileFixed {
    static constexpr bool FIXED = true;
    static constexpr uint32_t kRS = R_ * S_;
    static constexpr uint32_t kLpp = C_ >= 32 ? 8 : C_ / 4;
    static constexpr uint32_t kLppLog = kLpp == 8 ? 3 : kLpp == 4 ? 2 : kLpp == 2 ? 1 : 0;
    static constexpr uint32_t kPsplit = (kRS + P_ - 1) / P_;
    static constexpr uint32_t kPp = (P_ + 31) / 32 * 32;
    static constexpr uint32_t kVpr = (P_ + 3) / 4;
    static constexpr uint32_t kCchunks = (C_ + 4 * kLpp - 1) / (4 * kLpp);
    __host__ __device__ static constexpr uint32_t nthr(const TileArgs&) { return NTHR_; }
    __host__ __device__ static constexpr uint32_t S(const TileArgs&) { return S_; }
    __host__ __device__ static constexpr uint32_t C(const TileArgs&) { return C_; }
    __host__ __device__ static constexpr uint32_t RS(const TileArgs&) { return kRS; }
    __host__ __device__ static constexpr uint32_t P(const TileArgs&) { return P_; }
    __host__ __device__ static constexpr uint32_t Pp(const TileArgs&) { return kPp; }
    __host__ __device__ static constexpr uint32_t psplit(const TileArgs&) { return kPsplit; }
    __host__ __device__ static constexpr uint32_t Ct(const TileArgs&) { return 4 * kLpp; }
    __host__ __device__ static constexpr uint32_t lppLog(const TileArgs&) { return kLppLog; }
    __host__ __device__ static constexpr uint32_t tpb(const TileArgs&) { return kPsplit * kCchunks; }
    __host__ __device__ static constexpr uint32_t vpr(const TileArgs&) { return kVpr; }
    __host__ __device__ static constexpr uint32_t divS(uint32_t v, const TileArgs&) { return v / (uint32_t)S_; }
    __host__ __device__ static constexpr uint32_t divPs(uint32_t v, const TileArgs&) { return v / kPsplit; }
    __host__ __device__ static constexpr uint32_t divTpb(uint32_t v, const TileArgs&) { return v / (kPsplit * kCchunks); }
    __host__ __device__ static constexpr uint32_t divVpr(uint32_t v, const TileArgs&) { return v / kVpr; }
};

template <typename G>
__device__ __forceinline__ void decode_tile(const TileArgs& a, TileId& t, uint32_t ib, uint32_t rem)
{
    t.ib = ib;
    const uint32_t cc = G::divPs(rem, a);
    const uint32_t pc = rem - cc * G::psplit(a);
    t.c0 = (int)(cc * G::Ct(a));
    t.ctEff = (int)min(G::Ct(a), G::C(a) - (uint32_t)t.c0);
    t.p0 = (int)(pc * G::P(a));
    t.Pn = (int)min(G::P(a), G::RS(a) - (uint32_t)t.p0);
}

__device__ __forceinline__ uint32_t lds_swz(uint32_t c) { return ((c >> 2) & 7u) << 2; }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits until every global store of
// the wave has been acknowledged (vmcnt(0)), which would drain the store queue once per tile.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 16-byte LDS read of 4 consecutive floats.  The promise of alignment has to be explicit: a plain vector
// load through a cast pointer was lowered to two 8-byte-pair reads, which serialise on the LDS banks.
__device__ __forceinline__ f4 lds_read4(const float* p)
{
    return *static_cast<const f4*>(__builtin_assume_aligned(p, 16));
}

// Raw buffer access (V# descriptors): 32-bit byte offsets from a wave-uniform base, and hardware range
// checking: a load whose offset is outside the descriptor returns 0, a store is dropped.  Lanes with
// nothing to do get the offset 0xFFFFFFFF instead of a branch, and the addressing needs no 64-bit
// per-lane arithmetic; the planar kernels spent more cycles computing addresses than waiting for memory.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
constexpr uint32_t BUF_OOB = 0xFFFFFFFFu;
constexpr int BUF_NT = 2;  // cache-policy operand of the buffer builtins: nontemporal

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <int VEC> __device__ __forceinline__ typename Vec<VEC>::type buf_load(rsrc_t r, uint32_t off);
template <> __device__ __forceinline__ f4 buf_load<4>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
}
template <> __device__ __forceinline__ f2 buf_load<2>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(f2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
}
template <> __device__ __forceinline__ float buf_load<1>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}

template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const f4& v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), r, off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const f2& v)
{
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2, v), r, off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const float& v)
{
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, off, 0, AUX);
}

// ---- NHWC stack <-> NHWC tensor with buffer addressing ------------------------------------------
//
// The row-segment copies again, for images and blocks below 2^30 floats (everything but the largest
// tensors; the kernels above remain for those): both sides go through range-checked descriptors, lanes
// with nothing to move get an out-of-range offset, and there is no control flow between the first load
// and the last store.  In the branchy version every conditional store was preceded by a full wait for
// outstanding memory operations, stores included, so the four stores of a lane went out one after the
// completion of the other.

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
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const int64_t imgFloats = (int64_t)a.g.H * a.g.W * a.g.C;
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * imgFloats : 0), o.valid ? (uint32_t)imgFloats * 4u : 0u);
    const rsrc_t yr = make_rsrc(y + (int64_t)ib * a.blockV * VEC, a.blockV * (uint32_t)(VEC * 4));
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;
    vec v[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        const uint32_t r = fdiv(e, a.dRow);
        const int j = (int)(e - r * a.rowV);
        const int hh = o.h0 + (int)r;
        const bool ok = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi;
        // (unsigned arithmetic: the value only matters when ok, and then it is the in-range offset)
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0) * (uint32_t)CV + (uint32_t)j) * (uint32_t)(VEC * 4);
        v[u] = buf_load<VEC>(xr, ok ? off : BUF_OOB);
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        buf_store<BUF_NT>(yr, e < a.blockV ? e * (uint32_t)(VEC * 4) : BUF_OOB, v[u]);
    }
}

template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_nhwc(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, NhwcArgs a, ColorArgs col)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);
    if (!o.valid) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, o, atomics)) return;
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const int64_t imgFloats = (int64_t)a.g.H * a.g.W * a.g.C;
    float* img = y + (int64_t)o.n * imgFloats;
    const rsrc_t yr = make_rsrc(img, (uint32_t)imgFloats * 4u);
    const rsrc_t sr = make_rsrc(ysrc + (int64_t)o.n * imgFloats, (uint32_t)imgFloats * 4u);  // what an add reads
    const rsrc_t xr = make_rsrc(x + (int64_t)ib * a.blockV * VEC, a.blockV * (uint32_t)(VEC * 4));
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;
    vec v[NHWC_UNR];
    uint32_t dst[NHWC_UNR];
    int32_t own[NHWC_UNR];
    const rsrc_t wr = make_rsrc(MODE == SCATTER_OWNED ? col.owner + (int64_t)o.n * a.g.H * a.g.W : nullptr,
                                MODE == SCATTER_OWNED ? (uint32_t)(a.g.H * a.g.W) * 4u : 0u);
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        const uint32_t r = fdiv(e, a.dRow);
        const int j = (int)(e - r * a.rowV);
        const int hh = o.h0 + (int)r;
        bool ok = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi;
        if (MODE == SCATTER_RANKED) ok = ok && !ranked_out(rank_bits(col, ib), r, fdiv((uint32_t)j, a.dCV), a.g);
        dst[u] = ok ? (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0) * (uint32_t)CV + (uint32_t)j) * (uint32_t)(VEC * 4)
                    : BUF_OOB;
        v[u] = buf_load<VEC>(xr, ok ? e * (uint32_t)(VEC * 4) : BUF_OOB);  // off-image parts are not read
        if (MODE == SCATTER_OWNED) {
            const uint32_t pix = (uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0 + fdiv((uint32_t)j, a.dCV);
            own[u] = __builtin_bit_cast(int32_t, buf_load<1>(wr, ok ? pix * 4u : BUF_OOB));
        }
    }
    if (MODE == SCATTER_OWNED) {
        // (an out-of-range owner read returns 0, which may equal ib: dst is BUF_OOB there already)
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, own[u] == (int32_t)ib ? dst[u] : BUF_OOB, v[u]);
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED) {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, dst[u], v[u]);
    } else if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
        vec cur[NHWC_UNR];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) cur[u] = buf_load<VEC>(sr, dst[u]);
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, dst[u], vadd(cur[u], v[u]));
    } else {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) {
            if (dst[u] != BUF_OOB) {
                float* d = img + (dst[u] >> 2);
#pragma unroll
                for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v[u], k));
            }
        }
    }
}

// NHWC side of a tile: thread tid owns channel vector cl = tid & (lpp-1) of pixels pl0 + u*step,
// u = 0 .. TILE_LD-1, pl0 = tid >> lppLog, step = nthr >> lppLog.  Walks those pixels keeping (r, s) by
// increments and hands each one's byte offset inside the image (or BUF_OOB), its pixel number h*W + w (only
// meaningful with an in-range offset) and its position (r, s) inside the block to `f(u, pl, off, pix, r, s)`.
template <int VEC, typename G, typename F>
__device__ __forceinline__ void nhwc_walk(const TileArgs& a, const TileId& t, const BlockOrigin& o, uint32_t tid,
                                          uint32_t nthr, F f)
{
    const uint32_t lppLog = G::lppLog(a), S = G::S(a), C = G::C(a);
    const uint32_t lppMask = (1u << lppLog) - 1u;
    const uint32_t step = nthr >> lppLog;
    const uint32_t stepR = G::divS(step, a), stepS = step - stepR * S;
    uint32_t pl = tid >> lppLog;
    const uint32_t c = (uint32_t)t.c0 + (tid & lppMask) * VEC;
    const uint32_t p = (uint32_t)t.p0 + pl;
    uint32_t r = G::divS(p, a), s = p - r * S;
    const bool cok = c < C;
#pragma unroll
    for (int u = 0; u < TILE_LD; ++u) {
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
        const bool ok = cok && pl < (uint32_t)t.Pn && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww) * C + c) * 4u;
        f(u, pl, ok ? off : BUF_OOB, (uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww, r, s);
        pl += step;
        r += stepR;
        s += stepS;
        if (s >= S) {
            s -= S;
            ++r;
        }
    }
}

// sparse_gather.cc:67-88 with transpose == true: y[ib, c, r, s] = x[n, h0+r, w0+s, c] or 0.
template <int VEC>
__device__ __forceinline__ void gather_planar_tile(const float* __restrict__ x, float* __restrict__ y,
                                                   const int16_t* __restrict__ idx, const TileArgs& a, float* lds,
                                                   uint32_t ib, uint32_t rem)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t tid = threadIdx.x, nthr = blockDim.x;
    const uint32_t RS = (uint32_t)(a.g.R * a.g.S);
    TileId t;
    decode_tile<TileRt>(a, t, ib, rem);
    const RawTriple raw = load_triple(idx, t.ib);
    if (beyond_count(a.g, t.ib)) return;
    const BlockOrigin o = origin_of(raw, a.g);
    // a block index outside [0, N) gets an empty descriptor: every load returns 0
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * a.imgFloats : 0), o.valid ? a.imgBytes : 0u);

    vec v[TILE_LD];
    uint32_t pls[TILE_LD];
    nhwc_walk<VEC, TileRt>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t, uint32_t, uint32_t) {
        v[u] = buf_load<VEC>(xr, off);
        pls[u] = pl;
    });

    // registers -> LDS, transposing: this thread's VEC channels go to VEC rows, pixel pl to column pl
    const uint32_t c0l = (tid & ((1u << a.lppLog) - 1u)) * VEC;
#pragma unroll
    for (int u = 0; u < TILE_LD; ++u) {
        if (pls[u] < (uint32_t)t.Pn) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const uint32_t c = c0l + k;
                lds[c * a.Pp + (pls[u] ^ lds_swz(c))] = vget(v[u], k);
            }
        }
    }
    lds_barrier();

    // LDS -> global, planar side.  Full slots in a flat, branch-free loop ...
    const rsrc_t yr = make_rsrc(y + ((int64_t)t.ib * a.g.C + t.c0) * RS + t.p0,
                                ((uint32_t)(t.ctEff - 1) * RS + (uint32_t)t.Pn) * 4u);
    const uint32_t slots = (uint32_t)t.ctEff * a.vpr;
    for (uint32_t base = 0; base < slots; base += 4 * nthr) {
        f4 q[4];
        uint32_t off[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = base + u * nthr + tid;
            const uint32_t c = fdiv(i, a.dVpr);
            const uint32_t e0 = 4u * (i - c * a.vpr);
            const bool full = i < slots && e0 + 4u <= (uint32_t)t.Pn;
            q[u] = lds_read4(lds + (full ? c * a.Pp + (e0 ^ lds_swz(c)) : 0u));
            off[u] = full ? (c * RS + e0) * 4u : BUF_OOB;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) buf_store<BUF_NT>(yr, off[u], q[u]);
    }
    // ... then the 1-3 floats that end a run whose length is not a multiple of 4, one row per thread
    const uint32_t tail = (uint32_t)t.Pn & 3u;
    if (tail && tid < (uint32_t)t.ctEff) {
        const uint32_t e0 = (uint32_t)t.Pn - tail;
        const f4 q = lds_read4(lds + tid * a.Pp + (e0 ^ lds_swz(tid)));
        const uint32_t off = (tid * RS + e0) * 4u;
        buf_store<0>(yr, off, q.x);
        if (tail > 1) buf_store<0>(yr, off + 4u, q.y);
        if (tail > 2) buf_store<0>(yr, off + 8u, q.z);
    }
}

template <int VEC>
__global__ __launch_bounds__(512) void k_gather_planar(const float* __restrict__ x, float* __restrict__ y,
                                                       const int16_t* __restrict__ idx, TileArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for_each_block_of_workgroup(a, a.tpb, [&](uint32_t ib, uint32_t rem) {
        gather_planar_tile<VEC>(x, y, idx, a, lds, ib, rem);
    });
}

// ---------------------------------------------------------------------------------------------
// Planar gather whose workgroups own whole 128-byte lines of the output
// ---------------------------------------------------------------------------------------------
//
// A write-only probe of the tile pattern above (32 runs of 243 floats at 729-float pitch, 4-byte
// aligned, first and last line of every run shared with another workgroup) reaches 3.5 TB/s; the same
// bytes written as whole, 16-byte aligned lines that belong to one workgroup each reach 5.9 TB/s.
// So this kernel cuts the output differently.  The Ct planes of a channel chunk are one contiguous
// piece of y, "the chunk", addressed by a linear float index l = c*RS + p.  Tile (chunk, split) still
// reads the pixels [p0, p1) for all Ct channels, but for row c it writes the lines that START inside
// [c*RS + p0, c*RS + p1): the range [up(c*RS + p0), up(c*RS + p1)), up() rounding to the next line of
// y (the two ends of the chunk stay where they are).  These ranges tile the chunk exactly, every store
// is an aligned dwordx4, and no line is written by two workgroups (except the one line two chunks may
// share).  The price is that a tile needs up to 31 pixels beyond p1 -- for the last split of a plane,
// where row c's last line runs into row c+1, the first 31 pixels of the plane -- so the tile's pixel
// window is [p0, p1 + LINE_EXT) taken cyclically over the plane, about 13 % more NHWC reads at 243
// pixels per tile; the extra pixels are read by the neighbouring tile as well and come from cache (a
// bare read-and-write of this access pattern takes the same time with and without them).  Used when a
// plane is split over several tiles; a tile of whole planes already writes one contiguous piece.
//
// LDS: row c at c*Pp, window pixel q at column q + phi(c), phi(c) = (c*RS + p0) & 3, XOR-swizzled as
// above.  The shift phi makes LDS columns congruent to l modulo 4, so every output slot is one
// ds_read_b128.  In the last split the wrapped pixels of channel c (the first pixels of its plane) are
// stored behind the pixels of channel c-1 instead, where l continues: the slots of row c-1's last line
// that cross into plane c are then contiguous in LDS like any other.

constexpr int LINE_FLOATS = 32;
constexpr int LINE_EXT = LINE_FLOATS - 1;

struct LineArgs {
    Geom g;
    int Ct, lppLog;
    int RS;
    int P, Pp, psplit, cchunks;
    int grid2d;         // the launch is (tpb, block rows): see for_each_block_of_workgroup
    uint32_t blocks;    // capacity of the block list (numActive)
    uint32_t tpb, total;
    uint32_t spr;       // bound on the output slots of one row of one tile
    int64_t imgFloats;
    uint32_t imgBytes;
    FastDiv dTpb, dPs, dS;
};

// Geometry of a launch as the kernels see it: either read from the argument struct (any shape) or fixed at compile
// time for the shapes the benchmark configurations use.  With constants the reciprocal divisions, the pitch
// multiplications and the pixel-step bookkeeping fold away (about a third of the vector instructions of a tile),
// LDS accesses take immediate offsets and the unused staging variants are not compiled in.  The host launches a
// fixed-shape instance only when the tile it chose equals the instance's (sbnet_launch.h: Geom::forceGeneric keeps
// tests on the run-time path).
struct LinesRt {
    static constexpr bool FIXED = false;
    __device__ static uint32_t nthr(const LineArgs&) { return blockDim.x; }
    __device__ static uint32_t R(const LineArgs& a) { return (uint32_t)a.g.R; }
    __device__ static uint32_t S(const LineArgs& a) { return (uint32_t)a.g.S; }
    __device__ static uint32_t C(const LineArgs& a) { return (uint32_t)a.g.C; }
    __device__ static uint32_t RS(const LineArgs& a) { return (uint32_t)a.RS; }
    __device__ static uint32_t P(const LineArgs& a) { return (uint32_t)a.P; }
    __device__ static uint32_t Pp(const LineArgs& a) { return (uint32_t)a.Pp; }
    __device__ static uint32_t psplit(const LineArgs& a) { return (uint32_t)a.psplit; }
    __device__ static uint32_t Ct(const LineArgs& a) { return (uint32_t)a.Ct; }
    __device__ static uint32_t lppLog(const LineArgs& a) { return (uint32_t)a.lppLog; }
    __device__ static uint32_t tpb(const LineArgs& a) { return a.tpb; }
    __device__ static uint32_t divS(uint32_t v, const LineArgs& a) { return fdiv(v, a.dS); }
    __device__ static uint32_t divPs(uint32_t v, const LineArgs& a) { return fdiv(v, a.dPs); }
    __device__ static uint32_t divTpb(uint32_t v, const LineArgs& a) { return fdiv(v, a.dTpb); }
};

template <int R_, int S_, int C_, int PSPLIT_, int NTHR_>
struct LinesFixed {
    static constexpr bool FIXED = true;
    static constexpr uint32_t kRS = R_ * S_;
    static constexpr uint32_t kLpp = C_ >= 32 ? 8 : C_ / 4;  // C_ a multiple of 4; Ct = min(C_, 32) rounded to 2^k*4
    static constexpr uint32_t kLppLog = kLpp == 8 ? 3 : kLpp == 4 ? 2 : kLpp == 2 ? 1 : 0;
    static constexpr uint32_t kP = (kRS + PSPLIT_ - 1) / PSPLIT_;
    static constexpr uint32_t kPp = (kP + LINE_EXT + 3 + 31) / 32 * 32;
    static constexpr uint32_t kCchunks = (C_ + 4 * kLpp - 1) / (4 * kLpp);
    static constexpr int kLD = (int)(((kP + LINE_EXT) * kLpp + NTHR_ - 1) / NTHR_) < 4
                                   ? 4 : (int)(((kP + LINE_EXT) * kLpp + NTHR_ - 1) / NTHR_);
    __host__ __device__ static constexpr uint32_t nthr(const LineArgs&) { return NTHR_; }
    __host__ __device__ static constexpr uint32_t R(const LineArgs&) { return R_; }
    __host__ __device__ static constexpr uint32_t S(const LineArgs&) { return S_; }
    __host__ __device__ static constexpr uint32_t C(const LineArgs&) { return C_; }
    __host__ __device__ static constexpr uint32_t RS(const LineArgs&) { return kRS; }
    __host__ __device__ static constexpr uint32_t P(const LineArgs&) { return kP; }
    __host__ __device__ static constexpr uint32_t Pp(const LineArgs&) { return kPp; }
    __host__ __device__ static constexpr uint32_t psplit(const LineArgs&) { return PSPLIT_; }
    __host__ __device__ static constexpr uint32_t Ct(const LineArgs&) { return 4 * kLpp; }
    __host__ __device__ static constexpr uint32_t lppLog(const LineArgs&) { return kLppLog; }
    __host__ __device__ static constexpr uint32_t tpb(const LineArgs&) { return PSPLIT_ * kCchunks; }
    __host__ __device__ static constexpr uint32_t divS(uint32_t v, const LineArgs&) { return v / (uint32_t)S_; }
    __host__ __device__ static constexpr uint32_t divPs(uint32_t v, const LineArgs&) { return v / (uint32_t)PSPLIT_; }
    __host__ __device__ static constexpr uint32_t divTpb(uint32_t v, const LineArgs&) { return v / (PSPLIT_ * kCchunks); }
};

template <int LD, typename G>
__device__ __forceinline__ void gather_lines_tile(const float* __restrict__ x, float* __restrict__ y,
                                                  const int16_t* __restrict__ idx, const LineArgs& a, float* lds,
                                                  uint32_t ib, uint32_t rem)
{
    const uint32_t tid = threadIdx.x, nthr = G::nthr(a);
    const uint32_t RS = G::RS(a), S = G::S(a), R = G::R(a), C = G::C(a), Pp = G::Pp(a);
    const uint32_t lppLog = G::lppLog(a);

    const RawTriple raw = load_triple(idx, ib);
    if (beyond_count(a.g, ib)) return;
    const uint32_t cc = G::divPs(rem, a);
    const uint32_t split = rem - cc * G::psplit(a);
    const uint32_t c0 = cc * G::Ct(a);
    const uint32_t ctEff = min(G::Ct(a), C - c0);
    const uint32_t p0 = split * G::P(a);
    const uint32_t p1 = min(p0 + G::P(a), RS);
    const uint32_t win = p1 - p0 + (uint32_t)LINE_EXT;

    const BlockOrigin o = origin_of(raw, a.g);
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * a.imgFloats : 0), o.valid ? a.imgBytes : 0u);

    // NHWC side: lane owns channels [4*cl, 4*cl + 4) of window pixels q0 + u*step.  (r, s) of the pixel is
    // kept by increments; stepping past the end of the plane wraps to its start, which is r -= R.
    const uint32_t cl = tid & ((1u << lppLog) - 1u);
    const uint32_t q0 = tid >> lppLog, step = nthr >> lppLog;
    const uint32_t c = c0 + cl * 4u;
    const bool cok = c < C;
    const uint32_t stepR = G::divS(step, a), stepS = step - stepR * S;
    uint32_t r, sc;
    {
        uint32_t p = p0 + q0;
        if (p >= RS) p -= RS;
        r = G::divS(p, a);
        sc = p - r * S;
    }
    f4 v[LD];
#pragma unroll
    for (int u = 0; u < LD; ++u) {
        const uint32_t q = q0 + (uint32_t)u * step;
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)sc;
        const bool ok = cok && q < win && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww) * C + c) * 4u;
        v[u] = buf_load<4>(xr, ok ? off : BUF_OOB);
        sc += stepS;
        r += stepR;
        if (sc >= S) {
            sc -= S;
            ++r;
        }
        if (r >= R) r -= R;
    }
    // registers -> LDS.  In the last split of a plane the window wraps: its pixels from `wrapStart` on are the
    // first pixels of the plane, which the output needs as the continuation of the PREVIOUS channel's row (the
    // last line of row c-1 runs into row c).  They are stored there, behind row c-1's own pixels, so that every
    // output slot is one aligned 16-byte LDS read; channel 0 of the chunk has no predecessor and drops them.
    const uint32_t wrapStart = (p1 == RS && p0 != 0u) ? RS - p0 : 0xFFFFFFFFu;
    if (wrapStart == 0xFFFFFFFFu) {
        // With a pixel step that is a multiple of 32 the swizzle (bits 2..4 of the column) does not depend on u,
        // and the column of (u, k) is the column of (0, k) plus u*step.
        const uint32_t swz = lds_swz(cl * 4u);
        uint32_t rowAddr[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t phi = ((uint32_t)k * RS + p0) & 3u;  // == ((4*cl + k)*RS + p0) & 3
            rowAddr[k] = (cl * 4u + (uint32_t)k) * Pp + phi;
        }
        if ((step & 31u) == 0) {
#pragma unroll
            for (int k = 0; k < 4; ++k) rowAddr[k] = (rowAddr[k] & ~3u) + (((rowAddr[k] & 3u) + q0) ^ swz);
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                if (q0 + (uint32_t)u * step < win) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) lds[rowAddr[k] + (uint32_t)u * step] = vget(v[u], k);
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                const uint32_t q = q0 + (uint32_t)u * step;
                if (q < win) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        lds[(rowAddr[k] & ~3u) + (((rowAddr[k] & 3u) + q) ^ swz)] = vget(v[u], k);
                }
            }
        }
    } else if ((step & 31u) == 0) {
        // the same with the wrapped pixels one row up: rows 4*cl+k-1 are this thread's own rows 4*cl+k-1 for
        // k >= 1 (same swizzle group), and row 4*cl-1 for k = 0
        const uint32_t swz = lds_swz(cl * 4u);
        uint32_t rowAddr[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t phi = ((uint32_t)k * RS + p0) & 3u;
            rowAddr[k] = (cl * 4u + (uint32_t)k) * Pp + ((phi + q0) ^ swz);
        }
        const uint32_t rowP = cl * 4u - 1u;  // no such row for cl == 0: channel 0 drops its wrapped pixels
        const uint32_t addrP = rowP * Pp + ((((rowP * RS + p0) & 3u) + q0) ^ lds_swz(rowP));
#pragma unroll
        for (int u = 0; u < LD; ++u) {
            const uint32_t q = q0 + (uint32_t)u * step;
            if (q < win) {
                const bool wr = q >= wrapStart;
                if (!(wr && cl == 0u)) lds[(wr ? addrP : rowAddr[0]) + (uint32_t)u * step] = vget(v[u], 0);
#pragma unroll
                for (int k = 1; k < 4; ++k) lds[(wr ? rowAddr[k - 1] : rowAddr[k]) + (uint32_t)u * step] = vget(v[u], k);
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < LD; ++u) {
            const uint32_t q = q0 + (uint32_t)u * step;
            if (q < win) {
                const uint32_t back = q >= wrapStart ? 1u : 0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t row = cl * 4u + (uint32_t)k - back;  // 0xFFFFFFFF for channel 0's wrapped pixels
                    const uint32_t phi = (row * RS + p0) & 3u;
                    if (row != 0xFFFFFFFFu) lds[row * Pp + ((phi + q) ^ lds_swz(row))] = vget(v[u], k);
                }
            }
        }
    }
    lds_barrier();

    // planar side: whole lines of the chunk
    const int64_t chunkBase = ((int64_t)ib * C + c0) * RS;
    const uint32_t chunkFloats = ctEff * RS;
    const uint32_t a0 = (uint32_t)(((reinterpret_cast<uintptr_t>(y) >> 2) + (uint64_t)chunkBase) & (LINE_FLOATS - 1));
    const rsrc_t yr = make_rsrc(y + chunkBase, chunkFloats * 4u);
    {
        // One wave per row, four rows in flight: everything about the row (its range [A, B) of whole lines,
        // its swizzle) is wave-uniform and stays on the scalar unit; a lane only adds 4*k.
        const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
        const uint32_t lane = tid & 63u, nwaves = nthr >> 6;
        for (uint32_t cr0 = wave; cr0 < ctEff; cr0 += 4u * nwaves) {
            for (uint32_t kb = 0; kb < a.spr; kb += 64u) {
                f4 qv[4];
                uint32_t off[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t cr = cr0 + (uint32_t)u * nwaves;
                    const uint32_t lin0 = cr * RS + p0, lin1 = cr * RS + p1;
                    const uint32_t A = (lin0 == 0) ? 0u : ((a0 + lin0 + LINE_EXT) & ~(uint32_t)LINE_EXT) - a0;
                    const uint32_t B = (cr >= ctEff)          ? 0u
                                       : (lin1 == chunkFloats) ? chunkFloats
                                                               : ((a0 + lin1 + LINE_EXT) & ~(uint32_t)LINE_EXT) - a0;
                    const uint32_t colBase = A - lin0 + (lin0 & 3u);  // multiple of 4 less than 36
                    const uint32_t k4 = 4u * (kb + lane);
                    const uint32_t l = A + k4;
                    const bool live = l < B;
                    // (a row's last line may run into the next plane: those pixels sit behind the row in LDS)
                    qv[u] = lds_read4(lds + (live ? cr * Pp + ((colBase + k4) ^ lds_swz(cr)) : 0u));
                    off[u] = live ? l * 4u : BUF_OOB;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) buf_store<BUF_NT>(yr, off[u], qv[u]);
            }
        }
    }
}

// Launch shapes of the tile kernels.  (tiles per block, block rows): the block is the workgroup's y id, so its
// index triple can be fetched from preloaded kernel arguments before anything else arrives.  With the block count
// in device memory the launch cannot be sized for it: it covers half of the list's capacity in block rows and a
// workgroup takes block y and, if that is below the count, block y + rows.  Lists are rarely more than half full
// (sparse blocks pay off below that), so a workgroup almost never takes a second block, and the workgroups
// of rows past the count, which leave after one scalar load, are halved (at capacity 1024 and 312 blocks 17 088
// of them cost the scatter 3.6 us).  Beyond 65 535 block rows the launch is linear over the tiles.
template <typename ARGS, typename F>
__device__ __forceinline__ void for_each_block_of_workgroup(const ARGS& a, uint32_t tpb, F tile)
{
    if (a.grid2d) {
        // (two calls, not a loop: around a loop the compiler kept the whole tile's address arithmetic live and
        // tripled the register count)
        tile(blockIdx.y, blockIdx.x);
        const uint32_t ib2 = blockIdx.y + gridDim.y;
        if (ib2 < a.blocks && !beyond_count(a.g, ib2)) {  // (the same for the whole workgroup)
            __syncthreads();                               // LDS is reused
            tile(ib2, blockIdx.x);
        }
    } else {
        const uint32_t ib = blockIdx.x / tpb;
        tile(ib, blockIdx.x - ib * tpb);
    }
}

template <int LD, typename G>
__global__ __launch_bounds__(512) void k_gather_lines(const float* __restrict__ x, float* __restrict__ y,
                                                      const int16_t* __restrict__ idx, LineArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for_each_block_of_workgroup(a, G::tpb(a), [&](uint32_t ib, uint32_t rem) {
        gather_lines_tile<LD, G>(x, y, idx, a, lds, ib, rem);
    });
}

// sparse_gather.cc:103-130 with transpose == true: the block stack is [blocks, C, R, S].
template <int VEC, int MODE, typename G>
__device__ __forceinline__ void scatter_planar_tile(const float* __restrict__ x, float* y, const float* ysrc,
                                                    const int16_t* __restrict__ idx, const TileArgs& a,
                                                    const ColorArgs& col, float* lds, uint32_t ib, uint32_t rem)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t tid = threadIdx.x, nthr = G::nthr(a);
    const uint32_t RS = G::RS(a), Pp = G::Pp(a), vpr = G::vpr(a);
    TileId t;
    decode_tile<G>(a, t, ib, rem);
    const RawTriple raw = load_triple(idx, t.ib);  // scalar load, needed only after the barrier
    if (beyond_count(a.g, t.ib)) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, origin_of(raw, a.g), atomics)) return;  // (here: before the loads)

    // global -> registers, planar side.  The last slot of a run, when partial, is read as the last 4 floats
    // of the run instead (overlapping its neighbour): no load leaves the run, no value needs fixing up.
    const rsrc_t xr = make_rsrc(x + ((int64_t)t.ib * G::C(a) + t.c0) * RS + t.p0,
                                ((uint32_t)(t.ctEff - 1) * RS + (uint32_t)t.Pn) * 4u);
    const uint32_t slots = (uint32_t)t.ctEff * vpr;
    if (t.Pn >= 4) {
        f4 val[TILE_LD];
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            const uint32_t i = u * nthr + tid;
            const uint32_t c = G::divVpr(i, a);
            const int e0 = min(4 * (int)(i - c * vpr), t.Pn - 4);
            val[u] = buf_load<4>(xr, i < slots ? (c * RS + (uint32_t)e0) * 4u : BUF_OOB);
        }
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            const uint32_t i = u * nthr + tid;
            if (i < slots) {
                const uint32_t c = G::divVpr(i, a);
                const int e0 = 4 * (int)(i - c * vpr);
                float* __restrict__ row = lds + c * Pp;
                if (e0 + 4 <= t.Pn) {
                    *reinterpret_cast<f4*>(row + ((uint32_t)e0 ^ lds_swz(c))) = val[u];
                } else if (e0 < t.Pn) {  // partial last slot: holds floats [Pn-4, Pn) of the run
                    const uint32_t t0 = (uint32_t)(t.Pn - 4);
                    row[(t0 + 0) ^ lds_swz(c)] = val[u].x;
                    row[(t0 + 1) ^ lds_swz(c)] = val[u].y;
                    row[(t0 + 2) ^ lds_swz(c)] = val[u].z;
                    row[(t0 + 3) ^ lds_swz(c)] = val[u].w;
                }
            }
        }
    } else {
        // A plane's last split can hold fewer pixels than one slot (the split width is rounded up to whole slots,
        // and 1-3 pixels may remain): one thread per row moves them float by float.
        if (tid < (uint32_t)t.ctEff) {
            for (int k = 0; k < t.Pn; ++k)
                lds[tid * Pp + ((uint32_t)k ^ lds_swz(tid))] = buf_load<1>(xr, (tid * RS + (uint32_t)k) * 4u);
        }
    }
    lds_barrier();

    // NHWC side: LDS -> base tensor; pixels outside the image are dropped (sparse_gather.cc:121)
    const BlockOrigin o = origin_of(raw, a.g);
    if (!o.valid) return;
    float* img = y + (int64_t)o.n * a.imgFloats;
    const rsrc_t yr = make_rsrc(img, a.imgBytes);
    const rsrc_t sr = make_rsrc(ysrc + (int64_t)o.n * a.imgFloats, a.imgBytes);  // what an add reads
    const uint32_t c0l = (tid & ((1u << G::lppLog(a)) - 1u)) * VEC;
    vec w[TILE_LD];
    uint32_t offs[TILE_LD];
    int32_t own[TILE_LD];
    const rsrc_t wr = make_rsrc(MODE == SCATTER_OWNED ? col.owner + (int64_t)o.n * a.g.H * a.g.W : nullptr,
                                MODE == SCATTER_OWNED ? (uint32_t)(a.g.H * a.g.W) * 4u : 0u);
    const uint32_t rbits = MODE == SCATTER_RANKED ? rank_bits(col, t.ib) : 0u;
    nhwc_walk<VEC, G>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t pix, uint32_t r, uint32_t sc) {
        if (MODE == SCATTER_RANKED && ranked_out(rbits, r, sc, a.g)) off = BUF_OOB;
        offs[u] = off;
        if (MODE == SCATTER_OWNED) own[u] = __builtin_bit_cast(int32_t, buf_load<1>(wr, off != BUF_OOB ? pix * 4u : BUF_OOB));
        w[u] = vzero<VEC>();
        if (off != BUF_OOB) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const uint32_t c = c0l + k;
                vset(w[u], k, lds[c * Pp + (pl ^ lds_swz(c))]);
            }
        }
    });
    if (MODE == SCATTER_OWNED) {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, own[u] == (int32_t)t.ib ? offs[u] : BUF_OOB, w[u]);
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED) {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, offs[u], w[u]);
    } else if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
        vec cur[TILE_LD];
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) cur[u] = buf_load<VEC>(sr, offs[u]);
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, offs[u], vadd(cur[u], w[u]));
    } else {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            if (offs[u] != BUF_OOB) {
                float* d = img + (offs[u] >> 2);
#pragma unroll
                for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(w[u], k));
            }
        }
    }
}

template <int VEC, int MODE, typename G>
__global__ __launch_bounds__(512) void k_scatter_planar(const float* __restrict__ x, float* y, const float* ysrc,
                                                        const int16_t* __restrict__ idx, TileArgs a, ColorArgs col)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for_each_block_of_workgroup(a, G::tpb(a), [&](uint32_t ib, uint32_t rem) {
        scatter_planar_tile<VEC, MODE, G>(x, y, ysrc, idx, a, col, lds, ib, rem);
    });
}

// Fallback for block planes of fewer than 4 pixels (1x1, 1x2, 1x3 ... blocks), where a dwordx4 slot does
// not fit into a planar run: one thread per stack element.  The channel index varies fastest across
// threads, so the NHWC side stays coalesced.
template <int MODE, bool GATHER>
__global__ __launch_bounds__(256) void k_planar_small(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, Geom g, int64_t total,
                                                      const int32_t* __restrict__ owner)
{
    const int RS = g.R * g.S;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int c = (int)(i % g.C);
        const int p = (int)((i / g.C) % RS);
        const int64_t ib = i / ((int64_t)g.C * RS);
        if (g.countDev && ib >= *g.countDev) continue;
        const int r = p / g.S, s = p - r * g.S;
        const BlockOrigin o = load_origin(idx, (uint32_t)ib, g);
        const int hh = o.h0 + r, ww = o.w0 + s;
        const bool in = o.valid && (unsigned)hh < (unsigned)g.H && (unsigned)ww < (unsigned)g.W;
        const int64_t pix = (((int64_t)o.n * g.H + hh) * g.W + ww) * g.C + c;
        const int64_t st = (ib * g.C + c) * RS + p;
        if (GATHER) {
            y[st] = in ? x[pix] : 0.f;
        } else if (in) {
            if (MODE == SCATTER_OWNED) {
                if (owner[((int64_t)o.n * g.H + hh) * g.W + ww] == (int32_t)ib) y[pix] = x[st];
            } else if (MODE == SCATTER_RANKED) {
                if (!ranked_out((uint32_t)owner[ib], (uint32_t)r, (uint32_t)s, g)) y[pix] = x[st];
            } else if (MODE == SCATTER_ASSIGN) y[pix] = x[st];
            else if (MODE == SCATTER_ADD) y[pix] = ysrc[pix] + x[st];
            else atomic_add_f32(y + pix, x[st]);
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

constexpr int POOL_LD = 8;  // loads in flight per lane

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

// ---------------------------------------------------------------------------------------------
// overlapping scatter-add without atomics: every output pixel is summed by one owner
// ---------------------------------------------------------------------------------------------
//
// With bstride < bsize a pixel is covered by up to ceil(R/U)*ceil(S/V) blocks.  Hardware fp32 atomics
// resolve that at roughly a tenth of the HBM rate (every contribution is a read-modify-write in L2) and
// in arbitrary order.  Given a little scratch memory the add is done by "pulling" instead:
//   1. k_pull_fill / k_pull_map   an inverse map (n, bh, bw) -> position ib in the active list;
//   2. k_pull_table               per active block, the active blocks that overlap it, sorted by ib;
//   3. k_scatter_pull             the workgroup of block ib walks its own pixels; a pixel belongs to the
//                                 lowest-ib block that covers it, and that owner reads the pixel once,
//                                 adds the contributions of all covering blocks in ascending ib order
//                                 and writes it once.
// Ascending ib is the order in which the sequential CPU functor accumulates (sparse_gather.cc:105-129),
// so the result is bit-identical to it and reproducible from run to run.  A block listed twice cannot
// be represented in the map; k_pull_map notices, and k_scatter_pull then falls back to hardware atomics
// for the whole launch (still correct, to rounding).

constexpr int PULL_STEPS = 3;    // 64-vector steps of one wave, all in flight together (1: 223 us, 2: 228, 3: 211, 4: 232
                                 // on the 16x16-at-stride-8, 256-channel workload; 5 and more run out of registers)
constexpr int PULL_CLASSES = 9;  // 3 row classes x 3 column classes of a block's pixels (see below)
constexpr int PULL_COVER = 4;    // at most 2 x 2 blocks cover a pixel
constexpr int PULL_TABLE_STRIDE = PULL_CLASSES * PULL_COVER * 2;  // ints per block

// With at most 2x2 blocks over a pixel, which blocks cover a pixel of block (bh, bw) depends only on the pixel's
// class: its row is among the first R-U rows (shared with the blocks one step up), among the rows from U on (one
// step down) or in between (this row of blocks only), and the same for columns.  The table holds, per block and
// class, the up to four active blocks that cover pixels of the class, sorted by list position, each as (position,
// packed grid offset): the main kernel needs no search, and the first entry names the pixel's owner.

struct PullArgs {
    Geom g;
    int bhMin, bwMin, nBH, nBW;  // extent of the inverse map: blocks that can touch the image
    int kh1, kw1;                // Kh - 1, Kw - 1
    uint32_t CV, rowV, blockV;   // vectors per pixel, per block row, per block
    uint32_t cpb, units;         // wave-units per block, in total
    FastDiv dCpb, dRow, dCV;
};

__global__ __launch_bounds__(256) void k_pull_fill(int32_t* __restrict__ map, int64_t n, int32_t* __restrict__ dup)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) map[i] = -1;
    if (blockIdx.x == 0 && threadIdx.x == 0) *dup = 0;
}

__device__ __forceinline__ int64_t pull_slot(const PullArgs& a, int n, int bh, int bw)
{
    if ((unsigned)n >= (unsigned)a.g.N) return -1;
    const int ih = bh - a.bhMin, iw = bw - a.bwMin;
    if ((unsigned)ih >= (unsigned)a.nBH || (unsigned)iw >= (unsigned)a.nBW) return -1;
    return ((int64_t)n * a.nBH + ih) * a.nBW + iw;
}

__global__ __launch_bounds__(256) void k_pull_map(const int16_t* __restrict__ idx, int numActive, PullArgs a,
                                                  int32_t* __restrict__ map, int32_t* __restrict__ dup)
{
    const int ib = (int)(blockIdx.x * 256 + threadIdx.x);
    if (ib >= numActive || (a.g.countDev && ib >= *a.g.countDev)) return;
    const int64_t slot = pull_slot(a, idx[(size_t)ib * 3], idx[(size_t)ib * 3 + 1], idx[(size_t)ib * 3 + 2]);
    if (slot < 0) return;  // this block cannot touch the image
    if (atomicCAS(map + slot, -1, ib) != -1) *dup = 1;
}

// One thread per (block, class): the up to four active blocks that cover the class's pixels, sorted by position.
__global__ __launch_bounds__(256) void k_pull_table(const int16_t* __restrict__ idx, int numActive, PullArgs a,
                                                    const int32_t* __restrict__ map, int32_t* __restrict__ table)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const int ib = (int)(t / PULL_CLASSES), cls = (int)(t % PULL_CLASSES);
    if (ib >= numActive || (a.g.countDev && ib >= *a.g.countDev)) return;
    const int n = idx[(size_t)ib * 3], bh = idx[(size_t)ib * 3 + 1], bw = idx[(size_t)ib * 3 + 2];
    const int rc = cls / 3, cc = cls - rc * 3;
    // a block one step up covers the first R-U rows only (row class 0), one step down the rows from U on (class 2)
    const int dhLo = rc == 0 ? -a.kh1 : 0, dhHi = rc == 2 ? a.kh1 : 0;
    const int dwLo = cc == 0 ? -a.kw1 : 0, dwHi = cc == 2 ? a.kw1 : 0;
    int ids[PULL_COVER], pks[PULL_COVER];
    int cnt = 0;
    if (pull_slot(a, n, bh, bw) >= 0) {
        for (int dh = dhLo; dh <= dhHi; ++dh)
            for (int dw = dwLo; dw <= dwHi; ++dw) {
                const int64_t slot = pull_slot(a, n, bh + dh, bw + dw);
                const int other = slot >= 0 ? map[slot] : -1;
                if (other < 0) continue;
                int k = cnt++;  // insertion sort
                while (k > 0 && ids[k - 1] > other) {
                    ids[k] = ids[k - 1];
                    pks[k] = pks[k - 1];
                    --k;
                }
                ids[k] = other;
                pks[k] = ((dh & 0xffff) << 16) | (dw & 0xffff);
            }
    }
    typedef int i4 __attribute__((ext_vector_type(4)));
    int e[PULL_COVER * 2];
#pragma unroll
    for (int k = 0; k < PULL_COVER; ++k) {
        e[2 * k] = k < cnt ? ids[k] : -1;
        e[2 * k + 1] = k < cnt ? pks[k] : 0;
    }
    i4* q = reinterpret_cast<i4*>(table + (size_t)ib * PULL_TABLE_STRIDE + cls * (PULL_COVER * 2));
    q[0] = (i4){e[0], e[1], e[2], e[3]};
    q[1] = (i4){e[4], e[5], e[6], e[7]};
}

// sparse_gather.cc:103-130 with add == true on overlapping blocks, NHWC stack.
template <int VEC>
__global__ __launch_bounds__(256) void k_scatter_pull(const float* __restrict__ x, float* __restrict__ y,
                                                      const int16_t* __restrict__ idx, PullArgs a,
                                                      const int32_t* __restrict__ table,
                                                      const int32_t* __restrict__ dup)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);  // ib is wave-uniform: scalar load
    if (!o.valid) return;
    const vec* __restrict__ xv = reinterpret_cast<const vec*>(x);
    vec* __restrict__ yv = reinterpret_cast<vec*>(y);

    if (*dup != 0) {
        // the list names a block twice: the map cannot represent it; hardware atomics for the whole launch
        for (int step = 0; step < PULL_STEPS; ++step) {
            const uint32_t e = (chunk * PULL_STEPS + step) * 64 + lane;
            if (e >= a.blockV) break;
            const uint32_t r = fdiv(e, a.dRow);
            const uint32_t j = e - r * a.rowV;
            const uint32_t s = fdiv(j, a.dCV);
            const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
            if ((unsigned)hh >= (unsigned)a.g.H || (unsigned)ww >= (unsigned)a.g.W) continue;
            vec* dst = yv + ((((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * a.CV + (j - s * a.CV));
            commit<VEC, SCATTER_ATOMIC>(dst, ld_stream(xv + ((size_t)ib * a.blockV + e)));
        }
        return;
    }

    // Phase 1: per vector, its class's table entries (two 16-byte loads from a table line that the whole block shares).
    const int32_t* __restrict__ t = table + (size_t)ib * PULL_TABLE_STRIDE;
    typedef int i4 __attribute__((ext_vector_type(4)));
    i4 ent[PULL_STEPS][2];
    uint32_t rr[PULL_STEPS], ss[PULL_STEPS], cvv[PULL_STEPS];
    bool in[PULL_STEPS];
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
        const uint32_t e = (chunk * PULL_STEPS + u) * 64 + lane;
        const uint32_t r = fdiv(e, a.dRow);
        const uint32_t j = e - r * a.rowV;
        const uint32_t s = fdiv(j, a.dCV);
        rr[u] = r;
        ss[u] = s;
        cvv[u] = j - s * a.CV;
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
        in[u] = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t rc = (int)r < a.g.R - a.g.U ? 0u : ((int)r >= a.g.U ? 2u : 1u);
        const uint32_t cc = (int)s < a.g.S - a.g.V ? 0u : ((int)s >= a.g.V ? 2u : 1u);
        const i4* q = reinterpret_cast<const i4*>(t + (in[u] ? (rc * 3u + cc) * (PULL_COVER * 2) : 0u));
        ent[u][0] = q[0];
        ent[u][1] = q[1];
    }
    // Phase 2: the owner of a pixel (the first of the blocks that cover it) reads the pixel and every contribution.
    vec acc[PULL_STEPS], val[PULL_STEPS][PULL_COVER];
    bool mine[PULL_STEPS], has[PULL_STEPS][PULL_COVER];
    int64_t dstOff[PULL_STEPS];
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
        const int id[PULL_COVER] = {ent[u][0].x, ent[u][0].z, ent[u][1].x, ent[u][1].z};
        const int pk[PULL_COVER] = {ent[u][0].y, ent[u][0].w, ent[u][1].y, ent[u][1].w};
        mine[u] = in[u] && id[0] == (int)ib;
        const int hh = o.h0 + (int)rr[u], ww = o.w0 + (int)ss[u];
        dstOff[u] = (((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * a.CV + cvv[u];
        // (loads under their own conditions: a load that no lane of the wave needs is skipped, and at one block
        // in four active most pixels have one or two contributions, not four)
        acc[u] = vzero<VEC>();
        if (mine[u]) acc[u] = ld_stream(yv + dstOff[u]);
#pragma unroll
        for (int k = 0; k < PULL_COVER; ++k) {
            has[u][k] = mine[u] && id[k] >= 0;
            const int rs = (int)rr[u] - (int)(int16_t)(pk[k] >> 16) * a.g.U;
            const int cs = (int)ss[u] - (int)(int16_t)(pk[k] & 0xffff) * a.g.V;
            const int64_t off = (int64_t)id[k] * a.blockV + (int64_t)rs * a.rowV + (int64_t)cs * a.CV + cvv[u];
            val[u][k] = vzero<VEC>();
            if (has[u][k]) val[u][k] = ld_stream(xv + off);
        }
    }
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
#pragma unroll
        for (int k = 0; k < PULL_COVER; ++k)
            if (has[u][k]) acc[u] = vadd(acc[u], val[u][k]);  // ascending list position: the CPU functor's order
        if (mine[u]) st_stream(yv + dstOff[u], acc[u]);
    }
}

// ---------------------------------------------------------------------------------------------
// flat copy (CopyTensorFunctor, sparse_gather.cc:135-142 / sparse_gather.cu:268-276)
// ---------------------------------------------------------------------------------------------

constexpr int COPY_UNR = 4;  // 16 KB per workgroup; 32 KB per workgroup measured 30 % slower

__global__ __launch_bounds__(256) void k_copy_v4(const f4* __restrict__ src, f4* __restrict__ dst, size_t n4)
{
    const size_t base = (size_t)blockIdx.x * (256 * COPY_UNR) + threadIdx.x;
    f4 v[COPY_UNR];
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        v[u] = (f4)(0.f);
        if (i < n4) v[u] = ld_stream(src + i);
    }
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        if (i < n4) st_stream(dst + i, v[u]);
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

constexpr int GRID_Y_MAX = 65535;

// One workgroup per tile, as (tiles per block, block rows) when the block count fits the y dimension of a launch;
// half as many rows as the list holds when the count is only known on the device (for_each_block_of_workgroup).
static dim3 tile_grid(int grid2d, uint32_t tpb, int numActive, uint32_t total, const Geom& g)
{
    if (!grid2d) return dim3(total);
    return dim3(tpb, (unsigned)(g.countDev && numActive > 1 ? (numActive + 1) / 2 : numActive));
}

static int pick_vec(const Geom& g, const void* a, const void* b)
{
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
    if (g.C % 4 == 0 && (bits & 15) == 0) return 4;
    if (g.C % 2 == 0 && (bits & 7) == 0) return 2;
    return 1;
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
    a.dCV = make_fastdiv((uint32_t)(g.C / vec));
    return true;
}

// 32-bit byte offsets inside one image and inside one block: the buffer-addressed NHWC kernels apply.
static bool nhwc_fits_buffers(const Geom& g)
{
    return (int64_t)g.H * g.W * g.C < (1ll << 30) && (int64_t)g.R * g.S * g.C < (1ll << 30);
}

// Chooses the tile and the workgroup size of the planar kernels; the grid is one workgroup per tile.
static bool make_tile_args(const Geom& g, int numActive, int vec, TileArgs& a, int& threads, size_t& ldsBytes,
                           unsigned& grid, int defaultLdsBudget)
{
    a.g = g;
    const int64_t RS64 = (int64_t)g.R * g.S;
    if (RS64 >= (1ll << 30)) return false;
    const int RS = (int)RS64;
    // channels per tile: 32 floats (one 128-byte line per pixel) unless C is smaller
    const int ctWant = 32;
    int lpp = 1;
    while (lpp * 2 * vec <= ctWant && lpp * vec < g.C) lpp *= 2;
    a.Ct = lpp * vec;
    a.lppLog = ilog2_floor((uint32_t)lpp);
    a.cchunks = (g.C + a.Ct - 1) / a.Ct;
    // Pixels per tile are bounded by the LDS budget and by the TILE_LD registers per thread that hold a
    // tile in flight on either side.  The smallest workgroup that takes a whole block plane wins.
    const int budget = defaultLdsBudget;
    int maxP = 0;
    threads = 0;
    for (int nthr = 64; nthr <= 512; nthr *= 2) {
        const int pLds = (budget / (4 * a.Ct)) / 32 * 32;
        const int pItems = TILE_LD * nthr / lpp;
        const int pSlots = (TILE_LD * nthr / a.Ct) * 4 - 3;
        maxP = pLds < pItems ? pLds : pItems;
        if (pSlots < maxP) maxP = pSlots;
        threads = nthr;
        if (maxP >= RS) break;
    }
    if (maxP < 1) return false;
    a.psplit = (RS + maxP - 1) / maxP;
    a.P = (RS + a.psplit - 1) / a.psplit;
    // whole dwordx4 slots per planar run where the limits allow: only a plane's last split then ends in a
    // partial slot
    if (a.psplit > 1 && ((a.P + 3) & ~3) <= maxP) a.P = (a.P + 3) & ~3;
    a.psplit = (RS + a.P - 1) / a.P;
    a.Pp = (a.P + 31) / 32 * 32;
    a.vpr = (uint32_t)((a.P + 3) / 4);
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (a.imgFloats >= (1ll << 30) || (int64_t)g.C * RS64 >= (1ll << 30)) return false;  // 32-bit byte offsets
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    a.tpb = (uint32_t)(a.psplit * a.cchunks);
    const uint64_t total = (uint64_t)numActive * a.tpb;
    if (total >= (1ull << 31)) return false;
    a.total = (uint32_t)total;
    a.dTpb = make_fastdiv(a.tpb);
    a.dPs = make_fastdiv((uint32_t)a.psplit);
    a.dS = make_fastdiv((uint32_t)g.S);
    a.dVpr = make_fastdiv(a.vpr);
    ldsBytes = (size_t)a.Ct * a.Pp * sizeof(float);
    if (ldsBytes > 64 * 1024) return false;
    grid = a.total;
    a.grid2d = numActive <= GRID_Y_MAX;
    a.blocks = (uint32_t)numActive;
    return true;
}

// Compute units of the current device (256 on MI355X), looked up once per device.
static int device_cus()
{
    static std::mutex mutex;
    static int cus[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return 256;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        cus[dev] = n;
    }
    return cus[dev];
}

// Tile of the planar scatter.  16 KB tiles suit a launch that keeps every compute unit busy for several
// rounds of workgroups; a launch of few workgroups finishes in one or two rounds, where the loads and the stores
// of one round do not overlap much, and does better with 24 KB tiles (800x800x128 tensor, 27x27 blocks:
// 9.08 -> 8.87 us at 58 blocks, 20.6 -> 19.9 us at 156, but 40.8 -> 41.4 us at 312).
constexpr int SCATTER_FEW_WGS_PER_CU = 22;

// `share`: the launch does work for one block in `share` only (the passes of an overlapping add).
static bool scatter_tile_args(const Geom& g, int numActive, int vec, TileArgs& a, int& threads, size_t& ldsBytes,
                              unsigned& grid, int share = 1)
{
    if (!make_tile_args(g, numActive, vec, a, threads, ldsBytes, grid, 16 * 1024)) return false;
    if (a.psplit > 1 && a.total / (uint32_t)share < (uint32_t)(SCATTER_FEW_WGS_PER_CU * device_cus())) {
        TileArgs b;
        int bt;
        size_t bl;
        unsigned bg;
        if (make_tile_args(g, numActive, vec, b, bt, bl, bg, 24 * 1024) && b.psplit < a.psplit) {
            a = b;
            threads = bt;
            ldsBytes = bl;
            grid = bg;
        }
    }
    return true;
}

// Tile choice of k_gather_lines.  Returns false where the kernel does not apply (the caller then uses
// k_gather_planar): y not 16-byte aligned, a last split shorter than the window extension, LDS.
static bool make_line_args(const Geom& g, int numActive, const float* y, LineArgs& a, int& threads, int& ld,
                           size_t& ldsBytes, unsigned& grid, int maxLd)
{
    if (g.C % 4 != 0 || (reinterpret_cast<uintptr_t>(y) & 15) != 0) return false;
    a.g = g;
    const int64_t RS64 = (int64_t)g.R * g.S;
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (RS64 < 4 || a.imgFloats >= (1ll << 30) || (int64_t)g.C * RS64 >= (1ll << 30)) return false;
    const int RS = (int)RS64;
    a.RS = RS;
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    int lpp = 1;
    while (lpp * 2 * 4 <= 32 && lpp * 4 < g.C) lpp *= 2;
    a.Ct = lpp * 4;
    a.lppLog = ilog2_floor((uint32_t)lpp);
    a.cchunks = (g.C + a.Ct - 1) / a.Ct;
    // The smallest workgroup whose LD vectors per thread cover a whole plane; otherwise 512 threads and as
    // few splits as the window (own pixels + LINE_EXT) allows within maxLd vectors per thread.
    threads = 0;
    a.psplit = 1;
    for (int nthr = 64; nthr <= 512; nthr *= 2) {
        threads = nthr;
        if (4 * nthr / lpp >= RS) break;
    }
    if (4 * threads / lpp < RS) {
        const int cap = maxLd * threads / lpp - LINE_EXT;
        if (cap < 2 * LINE_FLOATS) return false;
        a.psplit = (RS + cap - 1) / cap;
    }
    a.P = (RS + a.psplit - 1) / a.psplit;
    a.psplit = (RS + a.P - 1) / a.P;
    // A tile that takes whole planes writes one contiguous piece of y in k_gather_planar already.
    if (a.psplit == 1) return false;
    if (RS - (a.psplit - 1) * a.P < LINE_FLOATS) return false;  // the last split must hold the extension
    const int win = a.P + LINE_EXT;
    ld = (win * lpp + threads - 1) / threads;
    if (ld < 4) ld = 4;
    if (ld > 8) return false;
    a.Pp = (win + 3 + 31) / 32 * 32;
    ldsBytes = (size_t)a.Ct * a.Pp * sizeof(float);
    if (ldsBytes > 64 * 1024) return false;
    // slots per row: the written range of a row is at most P + LINE_EXT floats; when every chunk starts on a
    // line it is a whole number of lines
    const bool aligned = (reinterpret_cast<uintptr_t>(y) & 127) == 0 && ((int64_t)a.Ct * RS) % LINE_FLOATS == 0 &&
                         ((int64_t)g.C * RS) % LINE_FLOATS == 0;
    a.spr = aligned ? (uint32_t)((a.P + LINE_EXT) / LINE_FLOATS * (LINE_FLOATS / 4)) : (uint32_t)((a.P + LINE_EXT + 3) / 4);
    a.tpb = (uint32_t)(a.psplit * a.cchunks);
    const uint64_t total = (uint64_t)numActive * a.tpb;
    if (total >= (1ull << 31)) return false;
    a.total = (uint32_t)total;
    a.dTpb = make_fastdiv(a.tpb);
    a.dPs = make_fastdiv((uint32_t)a.psplit);
    a.dS = make_fastdiv((uint32_t)g.S);
    grid = a.total;
    a.grid2d = numActive <= GRID_Y_MAX;
    a.blocks = (uint32_t)numActive;
    return true;
}

// 5 vectors per thread (three splits of a 27x27 plane) for launches of many workgroups, 7 (two splits: fewer
// window pixels read twice, more bytes in flight per workgroup) for launches of few, as for the scatter:
// 8.62 -> 7.76 us at 58 blocks, 21.7 -> 20.8 us at 156, but 31.1 -> 31.6 us at 231 and 40.3 -> 40.6 us at 312.
constexpr int GATHER_FEW_WGS_PER_CU = 9;

static bool choose_line_args(const Geom& g, int numActive, const float* y, LineArgs& a, int& threads, int& ld,
                             size_t& ldsBytes, unsigned& grid)
{
    if (!make_line_args(g, numActive, y, a, threads, ld, ldsBytes, grid, 5)) return false;
    if (a.total < (uint32_t)(GATHER_FEW_WGS_PER_CU * device_cus())) {
        LineArgs b;
        int bt, bld;
        size_t bl;
        unsigned bg;
        if (make_line_args(g, numActive, y, b, bt, bld, bl, bg, 7) && b.psplit < a.psplit) {
            a = b;
            threads = bt;
            ld = bld;
            ldsBytes = bl;
            grid = bg;
        }
    }
    return true;
}

// Fixed-shape instances: launched when the run-time tile choice equals the instance's.
template <typename G>
static bool lines_match(const LineArgs& a, int threads, int ld)
{
    return !a.g.forceGeneric && a.g.R * a.g.S == (int)G::kRS && a.g.S == (int)G::S(a) && a.g.C == (int)G::C(a) &&
           a.psplit == (int)G::psplit(a) && threads == (int)G::nthr(a) && a.P == (int)G::kP && a.Pp == (int)G::kPp &&
           a.Ct == (int)G::Ct(a) && a.lppLog == (int)G::kLppLog && ld == G::kLD && a.tpb == G::tpb(a);
}

template <typename G>
static bool launch_fixed_lines_one(const float* x, float* y, const int16_t* idx, const LineArgs& a, int threads, int ld,
                                   size_t lds, int numActive, hipStream_t stream)
{
    if (!lines_match<G>(a, threads, ld)) return false;
    hipLaunchKernelGGL((k_gather_lines<G::kLD, G>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads), lds,
                       stream, x, y, idx, a);
    return true;
}

static bool launch_fixed_lines(const float* x, float* y, const int16_t* idx, const LineArgs& a, int threads, int ld,
                               size_t lds, int numActive, hipStream_t stream)
{
    // 27x27 blocks of 128 channels (800x800x128 tensor): three and two splits per plane; 18x18 blocks of 64 channels
    return launch_fixed_lines_one<LinesFixed<27, 27, 128, 3, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream) ||
           launch_fixed_lines_one<LinesFixed<27, 27, 128, 2, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream) ||
           launch_fixed_lines_one<LinesFixed<18, 18, 64, 2, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream);
}

template <typename G>
static bool tile_match(const TileArgs& a, int threads)
{
    return !a.g.forceGeneric && a.g.R * a.g.S == (int)G::kRS && a.g.S == (int)G::S(a) && a.g.C == (int)G::C(a) &&
           a.P == (int)G::P(a) && a.psplit == (int)G::kPsplit && threads == (int)G::nthr(a) && a.Pp == (int)G::kPp &&
           a.Ct == (int)G::Ct(a) && a.lppLog == (int)G::kLppLog && a.vpr == G::kVpr && a.tpb == G::tpb(a);
}

template <int VEC, int MODE, typename G>
static bool launch_fixed_scatter_one(const float* x, float* y, const float* ysrc, const int16_t* idx, const TileArgs& a,
                                     int threads, size_t lds, int numActive, const ColorArgs& aux, hipStream_t stream)
{
    if (!tile_match<G>(a, threads)) return false;
    hipLaunchKernelGGL((k_scatter_planar<VEC, MODE, G>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads),
                       lds, stream, x, y, ysrc, idx, a, aux);
    return true;
}

template <int VEC, int MODE>
static bool launch_fixed_scatter(const float* x, float* y, const float* ysrc, const int16_t* idx, const TileArgs& a,
                                 int threads, size_t lds, int numActive, const ColorArgs& aux, hipStream_t stream)
{
    if constexpr (VEC == 4 && (MODE == SCATTER_ASSIGN || MODE == SCATTER_ADD || MODE == SCATTER_RANKED)) {
        // 27x27 blocks of 128 channels with 16 KB and 24 KB tiles; 16x16 blocks of 64 channels
        return launch_fixed_scatter_one<VEC, MODE, TileFixed<27, 27, 128, 124, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                      numActive, aux, stream) ||
               launch_fixed_scatter_one<VEC, MODE, TileFixed<27, 27, 128, 184, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                      numActive, aux, stream) ||
               launch_fixed_scatter_one<VEC, MODE, TileFixed<16, 16, 64, 128, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                     numActive, aux, stream);
    }
    return false;
}

template <int VEC>
static void gather_dispatch(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive,
                            bool transpose, hipStream_t stream, hipError_t& err)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        if (nhwc_fits_buffers(g))
            hipLaunchKernelGGL(k_gather_nhwc<VEC>, dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
        else
            hipLaunchKernelGGL(k_gather_nhwc_wide<VEC>, dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        if (VEC == 4) {
            LineArgs la;
            int ld;
            if (choose_line_args(g, numActive, y, la, threads, ld, lds, grid)) {
                if (launch_fixed_lines(x, y, idx, la, threads, ld, lds, numActive, stream)) return;
                const dim3 lg = tile_grid(la.grid2d, la.tpb, numActive, la.total, la.g);
                switch (ld) {
                case 4: hipLaunchKernelGGL((k_gather_lines<4, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 5: hipLaunchKernelGGL((k_gather_lines<5, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 6: hipLaunchKernelGGL((k_gather_lines<6, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 7: hipLaunchKernelGGL((k_gather_lines<7, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                default: hipLaunchKernelGGL((k_gather_lines<8, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                }
                return;
            }
        }
        // 32 KB tiles: 46.5 us against 52.7 us with 16 KB tiles on the 800x800x128 workload.
        // Planes of fewer than 4 pixels and images or blocks beyond 32-bit byte offsets take the generic kernel.
        if ((int64_t)g.R * g.S < 4 || !make_tile_args(g, numActive, VEC, a, threads, lds, grid, 32 * 1024)) {
            const int64_t total = (int64_t)numActive * g.C * g.R * g.S;
            const int64_t wgs = (total + 255) / 256;
            hipLaunchKernelGGL((k_planar_small<SCATTER_ASSIGN, true>), dim3((unsigned)(wgs > 65536 ? 65536 : wgs)),
                               dim3(256), 0, stream, x, y, (const float*)y, idx, g, total, (const int32_t*)nullptr);
            return;
        }
        hipLaunchKernelGGL(k_gather_planar<VEC>, tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads), lds,
                           stream, x, y, idx, a);
    }
}

// Test hook (sbnet_test_tile_choice): the tile the planar kernels would use for a geometry, without launching.
// kind 0: k_gather_lines, 1: k_gather_planar, 2: k_scatter_planar.  out = {threads, ldsBytes, P, Pp, psplit, Ct,
// cchunks, vectors or slots per thread needed, vectors or slots per thread available, last split's pixels, fixed
// instance available}.  Returns 0 when that kernel does not apply to the geometry.
int tile_choice(int kind, const Geom& g, int numActive, int vec, int yAlignedTo, int32_t* out)
{
    int threads = 0;
    size_t lds = 0;
    unsigned grid = 0;
    const int RS = g.R * g.S;
    if (kind == 0) {
        LineArgs a;
        int ld = 0;
        // a y pointer with the requested alignment (never dereferenced)
        const float* y = reinterpret_cast<const float*>((uintptr_t)0x10000 + (uintptr_t)yAlignedTo);
        if (vec != 4 || !choose_line_args(g, numActive, y, a, threads, ld, lds, grid)) return 0;
        const int lpp = 1 << a.lppLog;
        out[0] = threads; out[1] = (int32_t)lds; out[2] = a.P; out[3] = a.Pp; out[4] = a.psplit; out[5] = a.Ct;
        out[6] = a.cchunks; out[7] = ((a.P + LINE_EXT) * lpp + threads - 1) / threads; out[8] = ld;
        out[9] = RS - (a.psplit - 1) * a.P;
        out[10] = lines_match<LinesFixed<27, 27, 128, 3, 512>>(a, threads, ld) ||
                  lines_match<LinesFixed<27, 27, 128, 2, 512>>(a, threads, ld) ||
                  lines_match<LinesFixed<18, 18, 64, 2, 512>>(a, threads, ld);
        return 1;
    }
    TileArgs a;
    if (RS < 4) return 0;
    if (kind == 1 ? !make_tile_args(g, numActive, vec, a, threads, lds, grid, 32 * 1024)
                  : !scatter_tile_args(g, numActive, vec, a, threads, lds, grid))
        return 0;
    const int lpp = 1 << a.lppLog;
    out[0] = threads; out[1] = (int32_t)lds; out[2] = a.P; out[3] = a.Pp; out[4] = a.psplit; out[5] = a.Ct;
    out[6] = a.cchunks;
    // per thread: NHWC items and planar slots of a full tile
    const int items = (a.P * lpp + threads - 1) / threads;
    const int slots = (int)((a.Ct * a.vpr + threads - 1) / threads);
    out[7] = items > slots || kind == 1 ? items : slots;   // the gather's planar side loops, only its NHWC side is bounded
    out[8] = TILE_LD;
    out[9] = RS - (a.psplit - 1) * a.P;
    out[10] = kind == 2 && vec == 4 &&
              (tile_match<TileFixed<27, 27, 128, 124, 512>>(a, threads) || tile_match<TileFixed<27, 27, 128, 184, 512>>(a, threads) ||
               tile_match<TileFixed<16, 16, 64, 128, 512>>(a, threads));
    return 1;
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

// `ysrc` is what an add reads: y itself for the in-place op, the base tensor when y is being built as
// "copy of the base + scatter" without copying the covered pixels first.
template <int VEC, int MODE>
static void scatter_dispatch(const float* x, float* y, const float* ysrc, const int16_t* idx, const Geom& g,
                             int numActive, bool transpose, hipStream_t stream, hipError_t& err,
                             const int32_t* order = nullptr)
{
    // `order`: the owner map (SCATTER_OWNED) or the rank table (SCATTER_RANKED)
    const ColorArgs aux{1, 1, 0, nullptr, MODE == SCATTER_OWNED ? order : nullptr,
                        MODE == SCATTER_RANKED ? order : nullptr};
    const int32_t* owner = order;
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        if (nhwc_fits_buffers(g))
            hipLaunchKernelGGL((k_scatter_nhwc<VEC, MODE>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, ysrc,
                               idx, a, aux);
        else
            hipLaunchKernelGGL((k_scatter_nhwc_wide<VEC, MODE>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y,
                               ysrc, idx, a, aux);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        // 16 KB tiles: 42.6 us against 43.9 us with 32 KB tiles on the same workload
        if ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, VEC, a, threads, lds, grid)) {
            const int64_t total = (int64_t)numActive * g.C * g.R * g.S;
            const int64_t wgs = (total + 255) / 256;
            hipLaunchKernelGGL((k_planar_small<MODE, false>), dim3((unsigned)(wgs > 65536 ? 65536 : wgs)), dim3(256),
                               0, stream, x, y, ysrc, idx, g, total, owner);
            return;
        }
        if (launch_fixed_scatter<VEC, MODE>(x, y, ysrc, idx, a, threads, lds, numActive, aux, stream)) return;
        hipLaunchKernelGGL((k_scatter_planar<VEC, MODE, TileRt>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g),
                           dim3(threads), lds, stream, x, y, ysrc, idx, a, aux);
    }
}

template <int VEC>
static void scatter_mode(const float* x, float* y, const float* ysrc, const int16_t* idx, const Geom& g, int numActive,
                         bool transpose, ScatterMode mode, hipStream_t stream, hipError_t& err, const int32_t* order,
                         bool ranked)
{
    if (mode == SCATTER_ASSIGN && order && ranked)
        scatter_dispatch<VEC, SCATTER_RANKED>(x, y, ysrc, idx, g, numActive, transpose, stream, err, order);
    else if (mode == SCATTER_ASSIGN && order)
        scatter_dispatch<VEC, SCATTER_OWNED>(x, y, ysrc, idx, g, numActive, transpose, stream, err, order);
    else if (mode == SCATTER_ASSIGN)
        scatter_dispatch<VEC, SCATTER_ASSIGN>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
    else if (mode == SCATTER_ADD)
        scatter_dispatch<VEC, SCATTER_ADD>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
    else
        scatter_dispatch<VEC, SCATTER_ATOMIC>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
}

static hipError_t scatter_from(const float* x, float* y, const float* ysrc, const int16_t* idx, int numActive,
                               const Geom& g, bool transpose, ScatterMode mode, hipStream_t stream,
                               const int32_t* order = nullptr, bool ranked = false)
{
    if (numActive == 0) return hipSuccess;
    hipError_t err = hipSuccess;
    int vec = pick_vec(g, y, transpose ? nullptr : x);
    const int vsrc = pick_vec(g, ysrc, nullptr);
    if (vsrc < vec) vec = vsrc;
    if (vec == 4) scatter_mode<4>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked);
    else if (vec == 2) scatter_mode<2>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked);
    else scatter_mode<1>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked);
    if (err != hipSuccess) return err;
    return hipGetLastError();
}

hipError_t launch_scatter(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                          bool transpose, ScatterMode mode, hipStream_t stream)
{
    return scatter_from(x, y, y, idx, numActive, g, transpose, mode, stream);
}

// Extent of the inverse block map (blocks that can touch the image); false when it cannot be built.
static bool make_map_args(const Geom& g, PullArgs& a, int64_t& mapN)
{
    a.g = g;
    // oh + bh*U + R - 1 >= 0 and oh + bh*U <= H - 1 (floor divisions)
    auto floordiv = [](int64_t p, int64_t q) { return p >= 0 ? p / q : -((-p + q - 1) / q); };
    int64_t bhMin = -floordiv((int64_t)g.R - 1 + g.oh, g.U), bhMax = floordiv((int64_t)g.H - 1 - g.oh, g.U);
    int64_t bwMin = -floordiv((int64_t)g.S - 1 + g.ow, g.V), bwMax = floordiv((int64_t)g.W - 1 - g.ow, g.V);
    if (bhMin < -32768) bhMin = -32768;
    if (bwMin < -32768) bwMin = -32768;
    if (bhMax > 32767) bhMax = 32767;
    if (bwMax > 32767) bwMax = 32767;
    if (bhMax < bhMin || bwMax < bwMin) return false;
    a.bhMin = (int)bhMin; a.bwMin = (int)bwMin;
    a.nBH = (int)(bhMax - bhMin + 1); a.nBW = (int)(bwMax - bwMin + 1);
    mapN = (int64_t)g.N * a.nBH * a.nBW;
    return mapN < (1ll << 31);
}

// Geometry of the pull scatter; false when the method does not apply.
static bool make_pull_args(const Geom& g, int numActive, int vec, PullArgs& a, int64_t& mapN)
{
    const int Kh = (g.R + g.U - 1) / g.U, Kw = (g.S + g.V - 1) / g.V;
    if (Kh > 2 || Kw > 2) return false;  // at most 2x2 blocks over a pixel: neighbours one step away only
    if (!make_map_args(g, a, mapN)) return false;
    a.kh1 = Kh - 1;
    a.kw1 = Kw - 1;
    const uint64_t rowV = (uint64_t)g.S * g.C / vec, blockV = rowV * g.R;
    if (blockV >= (1ull << 31)) return false;
    a.CV = (uint32_t)(g.C / vec);
    a.rowV = (uint32_t)rowV;
    a.blockV = (uint32_t)blockV;
    a.cpb = (uint32_t)((blockV + 64 * PULL_STEPS - 1) / (64 * PULL_STEPS));
    const uint64_t units = (uint64_t)numActive * a.cpb;
    if (units >= (1ull << 31)) return false;
    a.units = (uint32_t)units;
    a.dCpb = make_fastdiv(a.cpb);
    a.dRow = make_fastdiv(a.rowV);
    a.dCV = make_fastdiv(a.CV);
    return true;
}

size_t scatter_pull_workspace_bytes(const Geom& g, int numActive)
{
    PullArgs a;
    int64_t mapN = 0;
    if (numActive <= 0 || !make_pull_args(g, numActive, 1, a, mapN)) return 0;
    return (size_t)mapN * 4 + 16 + 16 + (size_t)numActive * PULL_TABLE_STRIDE * 4;  // map, flag, alignment, table
}

hipError_t launch_scatter_pull(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                               void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (numActive == 0) { done = true; return hipSuccess; }
    PullArgs a;
    int64_t mapN = 0;
    const int vec = pick_vec(g, y, x);
    if (!workspace || !make_pull_args(g, numActive, vec, a, mapN)) return hipSuccess;
    if (workspaceBytes < scatter_pull_workspace_bytes(g, numActive) || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return hipSuccess;
    int32_t* map = static_cast<int32_t*>(workspace);
    int32_t* dup = map + mapN;
    // the table is read with 16-byte loads
    int32_t* table = reinterpret_cast<int32_t*>((reinterpret_cast<uintptr_t>(dup + 4) + 15) & ~(uintptr_t)15);
    int64_t fillWgs = (mapN + 255) / 256;
    if (fillWgs > 4096) fillWgs = 4096;
    if (fillWgs < 1) fillWgs = 1;
    const unsigned perBlockWgs = (unsigned)((numActive + 255) / 256);
    hipLaunchKernelGGL(k_pull_fill, dim3((unsigned)fillWgs), dim3(256), 0, stream, map, mapN, dup);
    hipLaunchKernelGGL(k_pull_map, dim3(perBlockWgs), dim3(256), 0, stream, idx, numActive, a, map, dup);
    hipLaunchKernelGGL(k_pull_table, dim3((unsigned)(((int64_t)numActive * PULL_CLASSES + 255) / 256)), dim3(256), 0,
                       stream, idx, numActive, a, map, table);
    const unsigned wgs = (a.units + 3) / 4;
    if (vec == 4) hipLaunchKernelGGL(k_scatter_pull<4>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    else if (vec == 2) hipLaunchKernelGGL(k_scatter_pull<2>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    else hipLaunchKernelGGL(k_scatter_pull<1>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    done = true;
    return hipGetLastError();
}

// ---- scatter-add in passes ------------------------------------------------------------------

constexpr int COLOR_MAX_PASSES = 16;

size_t scatter_color_workspace_bytes(const Geom& g, int numActive)
{
    PullArgs a;
    int64_t mapN = 0;
    const int64_t Kh = ((int64_t)g.R + g.U - 1) / g.U, Kw = ((int64_t)g.S + g.V - 1) / g.V;
    if (numActive <= 0 || Kh * Kw > COLOR_MAX_PASSES || !make_map_args(g, a, mapN)) return 0;
    return (size_t)mapN * 4 + 16;
}

template <int VEC>
static bool color_passes(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive, bool transpose,
                         ColorArgs col, int passes, hipStream_t stream)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) return false;
        const bool buf = nhwc_fits_buffers(g);
        for (col.pass = 0; col.pass < passes; ++col.pass) {
            if (buf)
                hipLaunchKernelGGL((k_scatter_nhwc<VEC, SCATTER_COLOR>), dim3((a.units + 3) / 4), dim3(256), 0, stream,
                                   x, y, (const float*)y, idx, a, col);
            else
                hipLaunchKernelGGL((k_scatter_nhwc_wide<VEC, SCATTER_COLOR>), dim3((a.units + 3) / 4), dim3(256), 0,
                                   stream, x, y, (const float*)y, idx, a, col);
        }
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        if ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, VEC, a, threads, lds, grid, passes)) return false;
        for (col.pass = 0; col.pass < passes; ++col.pass)
            hipLaunchKernelGGL((k_scatter_planar<VEC, SCATTER_COLOR, TileRt>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g),
                               dim3(threads), lds, stream, x, y, (const float*)y, idx, a, col);
    }
    return true;
}

hipError_t launch_scatter_colored(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                  bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream,
                                  bool& done)
{
    done = false;
    if (numActive == 0) { done = true; return hipSuccess; }
    const size_t need = scatter_color_workspace_bytes(g, numActive);
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return hipSuccess;
    PullArgs pa;
    int64_t mapN = 0;
    if (!make_map_args(g, pa, mapN)) return hipSuccess;
    ColorArgs col;
    col.kh = (g.R + g.U - 1) / g.U;
    col.kw = (g.S + g.V - 1) / g.V;
    col.pass = 0;
    int32_t* map = static_cast<int32_t*>(workspace);
    int32_t* dup = map + mapN;
    col.dup = dup;
    // geometry checks first: nothing is launched unless the passes can run
    const int vec = pick_vec(g, y, transpose ? nullptr : x);
    {
        NhwcArgs na;
        TileArgs ta;
        int threads;
        size_t lds;
        unsigned grid;
        if (!transpose ? !make_nhwc_args(g, numActive, vec, na)
                       : ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, vec, ta, threads, lds, grid, col.kh * col.kw)))
            return hipSuccess;
    }
    int64_t fillWgs = (mapN + 255) / 256;
    if (fillWgs > 4096) fillWgs = 4096;
    if (fillWgs < 1) fillWgs = 1;
    hipLaunchKernelGGL(k_pull_fill, dim3((unsigned)fillWgs), dim3(256), 0, stream, map, mapN, dup);
    hipLaunchKernelGGL(k_pull_map, dim3((unsigned)((numActive + 255) / 256)), dim3(256), 0, stream, idx, numActive, pa,
                       map, dup);
    const int passes = col.kh * col.kw;
    if (vec == 4) color_passes<4>(x, y, idx, g, numActive, transpose, col, passes, stream);
    else if (vec == 2) color_passes<2>(x, y, idx, g, numActive, transpose, col, passes, stream);
    else color_passes<1>(x, y, idx, g, numActive, transpose, col, passes, stream);
    done = true;
    return hipGetLastError();
}

// ---- "copy of the base + scatter" without copying what the scatter overwrites -------------------
//
// sparse_scatter (not the in-place op) returns a fresh tensor: the base, with the blocks written or added on
// top (sparse_gather.cc:338-346 copies the whole base, then scatters).  Copy-then-scatter moves every
// covered pixel twice more than needed.  With one flag byte per pixel ("an active block covers it") the work
// splits into two disjoint parts: k_copy_uncovered copies the pixels without the flag, and the ordinary
// scatter kernels write the flagged ones, reading the base (`ysrc`) where they add.  Same result, every byte
// moved once.  The flags cost N*H*W bytes of scratch and two small launches (clear, mark).

struct CoverArgs {
    Geom g;
    uint32_t RS;
    uint32_t imgV;      // vectors per image
    uint32_t imgBytes;
    int64_t imgFloats, imgPixels;
    FastDiv dCV, dS;
};

constexpr int COVER_UNR = 4;

__global__ __launch_bounds__(256) void k_cover_clear(uint32_t* __restrict__ words, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) words[i] = 0u;
}

// One thread per (block, block pixel): flags the pixel if it lies inside the image.  Blocks past the device-
// resident count and rows with an image number outside [0, N) flag nothing, as they scatter nothing.
__global__ __launch_bounds__(256) void k_cover_mark(const int16_t* __restrict__ idx, int numActive, CoverArgs a,
                                                    uint8_t* __restrict__ flags)
{
    const int64_t total = (int64_t)numActive * a.RS;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const uint32_t ib = (uint32_t)(i / a.RS);
        if (a.g.countDev && ib >= (uint32_t)*a.g.countDev) return;
        const uint32_t p = (uint32_t)(i - (int64_t)ib * a.RS);
        const uint32_t r = fdiv(p, a.dS), sc = p - r * (uint32_t)a.g.S;
        const BlockOrigin o = load_origin(idx, ib, a.g);
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)sc;
        if (o.valid && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W)
            flags[(int64_t)o.n * a.imgPixels + (int64_t)hh * a.g.W + ww] = 1;
    }
}

// Owner map of the ordered plain scatter (SCATTER_OWNED): -1 everywhere, then the highest list position among the
// blocks that cover each pixel.  Rows past the device-resident count and rows that name no image mark nothing.
__global__ __launch_bounds__(256) void k_owner_fill(int32_t* __restrict__ owner, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) owner[i] = -1;
}

__global__ __launch_bounds__(256) void k_owner_mark(const int16_t* __restrict__ idx, int numActive, CoverArgs a,
                                                    int32_t* __restrict__ owner)
{
    const int64_t total = (int64_t)numActive * a.RS;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const uint32_t ib = (uint32_t)(i / a.RS);
        if (a.g.countDev && ib >= (uint32_t)*a.g.countDev) return;
        const uint32_t p = (uint32_t)(i - (int64_t)ib * a.RS);
        const uint32_t r = fdiv(p, a.dS), sc = p - r * (uint32_t)a.g.S;
        const BlockOrigin o = load_origin(idx, ib, a.g);
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)sc;
        if (o.valid && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W)
            atomicMax(owner + ((int64_t)o.n * a.imgPixels + (int64_t)hh * a.g.W + ww), (int32_t)ib);
    }
}

// FLAG is the per-pixel coverage record: one byte (non-zero = covered), or the int32 owner map (>= 0 = covered).
template <int VEC, typename FLAG>
__global__ __launch_bounds__(256) void k_copy_uncovered(const float* __restrict__ src, float* __restrict__ dst,
                                                        const FLAG* __restrict__ flags, CoverArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t n = blockIdx.y;
    const rsrc_t sr = make_rsrc(src + (int64_t)n * a.imgFloats, a.imgBytes);
    const rsrc_t dr = make_rsrc(dst + (int64_t)n * a.imgFloats, a.imgBytes);
    const FLAG* __restrict__ fl = flags + (int64_t)n * a.imgPixels;
    const uint32_t e0 = blockIdx.x * (256u * COVER_UNR) + threadIdx.x;
    bool cov[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) {
        const uint32_t e = min(e0 + (uint32_t)u * 256u, a.imgV - 1u);
        const FLAG f = fl[fdiv(e, a.dCV)];
        cov[u] = sizeof(FLAG) == 1 ? f != 0 : (int32_t)f >= 0;
    }
    uint32_t off[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) {
        const uint32_t e = e0 + (uint32_t)u * 256u;
        off[u] = (e >= a.imgV || cov[u]) ? BUF_OOB : e * (uint32_t)(VEC * 4);
    }
    vec v[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) v[u] = buf_load<VEC>(sr, off[u]);
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) buf_store<BUF_NT>(dr, off[u], v[u]);
}

size_t scatter_cover_workspace_bytes(const Geom& g, int numActive)
{
    if (numActive <= 0) return 0;
    if ((int64_t)g.H * g.W * g.C >= (1ll << 30)) return 0;  // 32-bit byte offsets inside one image
    if ((int64_t)g.R * g.S >= (1ll << 31)) return 0;
    return (((size_t)g.N * g.H * g.W + 3) & ~(size_t)3) + 16;
}

static void make_cover_args(const Geom& g, int vec, CoverArgs& c)
{
    c.g = g;
    c.RS = (uint32_t)(g.R * g.S);
    c.imgFloats = (int64_t)g.H * g.W * g.C;
    c.imgPixels = (int64_t)g.H * g.W;
    c.imgV = (uint32_t)(c.imgFloats / vec);
    c.imgBytes = (uint32_t)(c.imgFloats * 4);
    c.dCV = make_fastdiv((uint32_t)(g.C / vec));
    c.dS = make_fastdiv((uint32_t)g.S);
}

// Nine bits per block for SCATTER_RANKED.  One wave per block: the lanes compare the block with every row of the
// list; a later row that names the same image and a grid position within one step in both directions sets the
// classes of pixels it shares with the block (itself included: a block listed twice loses all its pixels to the
// later row).
constexpr int RANK_MAX_BLOCKS = 4096;   // rows compared pairwise: 16.8 M comparisons at most

__global__ __launch_bounds__(256) void k_rank_table(const int16_t* __restrict__ idx, int numActive, Geom g,
                                                    int32_t* __restrict__ table)
{
    const uint32_t lane = threadIdx.x & 63u;
    const int ib = (int)(blockIdx.x * 4u + (threadIdx.x >> 6));
    int count = numActive;
    if (g.countDev) count = min(count, *g.countDev);
    if (ib >= count) return;
    const int n = idx[(size_t)ib * 3], bh = idx[(size_t)ib * 3 + 1], bw = idx[(size_t)ib * 3 + 2];
    uint32_t bits = 0u;
    for (int j = ib + 1 + (int)lane; j < count; j += 64) {
        const int dn = idx[(size_t)j * 3] - n, dh = idx[(size_t)j * 3 + 1] - bh, dw = idx[(size_t)j * 3 + 2] - bw;
        if (dn == 0 && dh >= -1 && dh <= 1 && dw >= -1 && dw <= 1) {
            // row classes (0: first R-U rows, 1: middle, 2: rows from U on) that a block dh steps away covers
            const uint32_t rows = dh < 0 ? 1u : (dh > 0 ? 4u : 7u), cols = dw < 0 ? 1u : (dw > 0 ? 4u : 7u);
#pragma unroll
            for (int rc = 0; rc < 3; ++rc)
                if (rows & (1u << rc)) bits |= cols << (3 * rc);
        }
    }
    for (int off = 32; off > 0; off >>= 1) bits |= (uint32_t)__shfl_xor((int)bits, off);
    if (lane == 0) table[ib] = (int32_t)bits;
}

// The rank table applies when at most 2x2 blocks share a pixel and the list is short enough for pairwise comparison.
static bool rank_table_applies(const Geom& g, int numActive)
{
    return numActive <= RANK_MAX_BLOCKS && g.R <= 2 * (int64_t)g.U && g.S <= 2 * (int64_t)g.V;
}

size_t scatter_owner_workspace_bytes(const Geom& g, int numActive)
{
    if (numActive <= 0 || !(g.U < g.R || g.V < g.S)) return 0;  // only overlapping blocks need an order
    if ((int64_t)g.R * g.S >= (1ll << 31)) return 0;
    // (the owner map; the rank table of the in-place op needs less, but the copying op always takes the map)
    const size_t map = (size_t)g.N * g.H * g.W * 4 + 16, table = (size_t)numActive * 4 + 16;
    return map > table ? map : table;
}

// Builds the owner map in `workspace`; false (nothing launched) when the ordered scatter does not apply.
static bool build_owner_map(const int16_t* idx, int numActive, const Geom& g, void* workspace, size_t workspaceBytes,
                            hipStream_t stream, int32_t*& owner)
{
    const size_t need = scatter_owner_workspace_bytes(g, numActive);
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3)) return false;
    owner = static_cast<int32_t*>(workspace);
    CoverArgs c;
    make_cover_args(g, 1, c);
    const int64_t n = (int64_t)g.N * g.H * g.W;
    int64_t wgs = (n + 1023) / 1024;
    if (wgs > 8192) wgs = 8192;
    hipLaunchKernelGGL(k_owner_fill, dim3((unsigned)wgs), dim3(256), 0, stream, owner, n);
    int64_t markWgs = ((int64_t)numActive * c.RS + 255) / 256;
    if (markWgs > 65536) markWgs = 65536;
    hipLaunchKernelGGL(k_owner_mark, dim3((unsigned)markWgs), dim3(256), 0, stream, idx, numActive, c, owner);
    return true;
}

hipError_t launch_scatter_owned(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (numActive == 0) { done = true; return hipSuccess; }
    if (rank_table_applies(g, numActive) && scatter_owner_workspace_bytes(g, numActive) != 0 && workspace &&
        workspaceBytes >= (size_t)numActive * 4 + 16 && (reinterpret_cast<uintptr_t>(workspace) & 3) == 0) {
        int32_t* table = static_cast<int32_t*>(workspace);
        hipLaunchKernelGGL(k_rank_table, dim3((unsigned)((numActive + 3) / 4)), dim3(256), 0, stream, idx, numActive, g,
                           table);
        done = true;
        return scatter_from(x, y, y, idx, numActive, g, transpose, SCATTER_ASSIGN, stream, table, true);
    }
    int32_t* owner = nullptr;
    if (!build_owner_map(idx, numActive, g, workspace, workspaceBytes, stream, owner)) return hipSuccess;
    done = true;
    return scatter_from(x, y, y, idx, numActive, g, transpose, SCATTER_ASSIGN, stream, owner);
}

hipError_t launch_scatter_over_base(const float* x, const float* ybase, float* y, const int16_t* idx, int numActive,
                                    const Geom& g, bool transpose, ScatterMode mode, void* workspace,
                                    size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (mode == SCATTER_ATOMIC || numActive <= 0) return hipSuccess;
    const size_t need = scatter_cover_workspace_bytes(g, numActive);
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return hipSuccess;
    // Two small launches prepare the flags: worth it once the blocks cover enough of the tensor to pay for them
    // (each covered byte saves one read and one write of the copy).
    if ((int64_t)numActive * g.R * g.S * g.C * 4 < (16ll << 20)) return hipSuccess;

    CoverArgs c;
    const int vec = pick_vec(g, ybase, y);
    make_cover_args(g, vec, c);
    const dim3 grid((c.imgV + 256u * COVER_UNR - 1) / (256u * COVER_UNR), (unsigned)g.N);

    // Plain writes of overlapping blocks: the owner map of the ordered scatter also tells which pixels are covered.
    if (mode == SCATTER_ASSIGN && scatter_owner_workspace_bytes(g, numActive) != 0) {
        int32_t* owner = nullptr;
        if (!build_owner_map(idx, numActive, g, workspace, workspaceBytes, stream, owner)) return hipSuccess;
        if (vec == 4) hipLaunchKernelGGL((k_copy_uncovered<4, int32_t>), grid, dim3(256), 0, stream, ybase, y, owner, c);
        else if (vec == 2) hipLaunchKernelGGL((k_copy_uncovered<2, int32_t>), grid, dim3(256), 0, stream, ybase, y, owner, c);
        else hipLaunchKernelGGL((k_copy_uncovered<1, int32_t>), grid, dim3(256), 0, stream, ybase, y, owner, c);
        done = true;
        return scatter_from(x, y, ybase, idx, numActive, g, transpose, mode, stream, owner);
    }
    uint8_t* flags = static_cast<uint8_t*>(workspace);

    const int64_t words = (int64_t)((need - 16) / 4);
    int64_t wgs = (words + 255) / 256;
    if (wgs > 8192) wgs = 8192;
    hipLaunchKernelGGL(k_cover_clear, dim3((unsigned)wgs), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(flags), words);
    int64_t markWgs = ((int64_t)numActive * c.RS + 255) / 256;
    if (markWgs > 65536) markWgs = 65536;
    hipLaunchKernelGGL(k_cover_mark, dim3((unsigned)markWgs), dim3(256), 0, stream, idx, numActive, c, flags);
    const uint8_t* cflags = flags;
    if (vec == 4) hipLaunchKernelGGL((k_copy_uncovered<4, uint8_t>), grid, dim3(256), 0, stream, ybase, y, cflags, c);
    else if (vec == 2) hipLaunchKernelGGL((k_copy_uncovered<2, uint8_t>), grid, dim3(256), 0, stream, ybase, y, cflags, c);
    else hipLaunchKernelGGL((k_copy_uncovered<1, uint8_t>), grid, dim3(256), 0, stream, ybase, y, cflags, c);
    done = true;
    return scatter_from(x, y, ybase, idx, numActive, g, transpose, mode, stream);
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
                               reinterpret_cast<const f4*>(src), reinterpret_cast<f4*>(dst), n4);
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
